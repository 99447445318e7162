// Direct-to-LDS MFMA GEMM kernel for gfx950: the fast path for shapes that are
// whole multiples of the workgroup tile.
//
// Differences from the register-staged kernel (gemm_kernel.hpp):
//   * operand tiles go global -> LDS with global_load_lds_dwordx4 (16 bytes per
//     lane, no VGPR round trip); a wave-level load always fills 1024 contiguous
//     LDS bytes in lane order, so each lane picks the GLOBAL address whose data
//     belongs in its fixed LDS slot (the swizzle is applied on the global side);
//   * an operand that is contiguous along M or N stays in that orientation in LDS
//     and is transposed on the way to registers by ds_read_b64_tr_b16;
//   * the LDS holds a ring of STAGES tiles; the loads of tile i+STAGES are issued as
//     soon as tile i's stage has been drained, so a load has STAGES-1 tile times to
//     land (measured: with one tile time the waves spend most of their cycles in
//     s_waitcnt vmcnt, and a pure load loop runs 25 % faster with two tiles in
//     flight than with one);
//   * MFMA operand registers are double-buffered across the 16-wide K steps of a
//     tile, and the one barrier per tile sits in front of the last K step, so its
//     cost and the next tile's first LDS reads hide under that step's MFMAs.
//
// LDS layouts (one operand tile = ROWS x BK 16-bit elements):
//   K-contiguous operand: row r = BK/8 chunks of 16 bytes; chunk c sits in slot
//     c ^ swizzle(r) (see swizzle_of_row).  Wave-level load t fills rows
//     t*512/BK .. (t+1)*512/BK - 1.
//   M/N-contiguous operand: 1024-byte blocks of 4 k-rows x 128 rows-of-the-tile;
//     block (kg, mh) at index kg * (ROWS/128) + mh; inside a block, k-row j holds
//     16 chunks of 8 elements, chunk c in slot c ^ (4*j) ^ (2*((kg/2)%2)).  Wave-level
//     load t fills block t.  ds_read_b64_tr_b16 then reads, per 32 lanes, either 4
//     k-rows x 32 elements of one block (32x32x16 MFMA) or 4 k-rows x 16 elements of
//     two blocks two k groups apart (16x16x32 MFMA) without bank conflicts
//     (measured for the first: 355 B/ns/CU vs 152 unswizzled).
//
// Same role as the staged kernel with respect to the reference (its gemm_impl,
// prefetch_fragment, load_matrix: reference kernel/kernel.hpp:108-556,
// kernel/load.hpp:348-966, kernel/fragment.hpp:191-274).
#ifndef ROCM_WMMA_GEMM_DIRECT_KERNEL_HPP
#define ROCM_WMMA_GEMM_DIRECT_KERNEL_HPP

#include <utility>

#include "gemm_kernel.hpp"

// Cache-policy bits of the global -> LDS loads (0 = default: cached in L1 and L2).
#ifndef RWG_LOAD_AUX
#define RWG_LOAD_AUX 0
#endif

namespace rocm_wmma_gemm
{
namespace device
{

typedef __fp16 fp16x4_raw __attribute__((__vector_size__(4 * sizeof(__fp16))));
using lds_char_ptr = __attribute__((address_space(3))) char*;

// One operand (A or B) of the direct pipeline.
//   ROWS   tile extent along M (for A) or N (for B)
//   WT     rows of the tile owned by one wave (wave tile extent)
//   WAVES  waves in the workgroup (all of them cooperate on every tile load)
//   MI     MFMA shape: 32 = v_mfma_f32_32x32x16 (lane l feeds row l%32, k 8*(l/32)..+7),
//                      16 = v_mfma_f32_16x16x32 (lane l feeds row l%16, k 8*(l/16)..+7)
template<bool KMAJOR, int ROWS, int BK, int WT, int WAVES, int MI = 32>
struct direct_operand
{
    static_assert(BK == 64 || BK == 32, "direct pipeline supports BK of 32 and 64");
    static_assert(MI == 32 || MI == 16, "MFMA shapes: 32x32x16 and 16x16x32");
    static constexpr int CH         = BK / 8; // 16-byte chunks per K-contiguous row
    static constexpr int KSTEP      = MI == 32 ? 16 : 32; // K extent of one MFMA
    static constexpr int KK         = BK / KSTEP; // MFMA K steps per tile
    static constexpr int TILE_BYTES = ROWS * BK * 2;
    static constexpr int LOADS      = TILE_BYTES / 1024; // wave-level loads per tile
    static_assert(LOADS % WAVES == 0, "tile loads must divide over the waves");
    static constexpr int PER_WAVE = LOADS / WAVES;
    static constexpr int T        = WT / MI; // MI-row MFMA operand tiles per wave
    static constexpr int MH       = ROWS / 128; // 128-row halves (M/N-contiguous layout)
    static constexpr int DS_PER_FRAGMENT = KMAJOR ? 1 : 2; // LDS reads behind one fragment()
    static constexpr int NOFF     = KMAJOR ? KK : T;
    static_assert(KMAJOR || ROWS % 128 == 0, "M/N-contiguous layout works in 128-row halves");

    // Per-lane element offset (from the tile origin at k = 0) of the 16 bytes this
    // lane fetches in the wave's i-th load; advancing a tile adds BK * stride_k.
    unsigned int lane_off[PER_WAVE];
    // Per-lane LDS byte offsets for fragment reads (within an operand tile).
    int frag_off[NOFF]; // K-contiguous: one per K step; M/N-contiguous: one per operand tile i

    __device__ __forceinline__ void init(int wave, int lane, long long ld, int wave_row0)
    {
#pragma unroll
        for(int i = 0; i < PER_WAVE; ++i)
        {
            const int t = wave + i * WAVES; // wave-level load index within the tile
            if constexpr(KMAJOR)
            {
                const int r    = (64 / CH) * t + lane / CH;
                const int slot = lane % CH;
                const int c    = slot ^ swizzle_of_row<CH, MI>(r);
                lane_off[i]    = (unsigned int)(r * ld + c * 8);
            }
            else
            {
                const int kg = t / MH, mh = t % MH;
                const int j = lane / 16, cphys = lane % 16;
                const int c = cphys ^ (4 * j) ^ (2 * ((kg >> 1) & 1));
                lane_off[i] = (unsigned int)((long long)(kg * 4 + j) * ld + mh * 128 + c * 8);
            }
        }
        if constexpr(KMAJOR)
        {
            // swizzle_of_row(row + 16*i) == swizzle_of_row(row)
            const int row = wave_row0 + (lane & (MI - 1));
            const int hi  = lane / MI; // which 8 k values of the K step this lane feeds
#pragma unroll
            for(int kk = 0; kk < KK; ++kk)
            {
                frag_off[kk] = row * (16 * CH)
                               + (((kk * (KSTEP / 8) + hi) ^ swizzle_of_row<CH, MI>(row)) * 16);
            }
        }
        else if constexpr(MI == 32)
        {
            const int b = lane / 16, s = lane % 16, j = s / 4;
#pragma unroll
            for(int i = 0; i < T; ++i)
            {
                const int m  = wave_row0 + i * 32 + 16 * (b % 2) + (s % 4) * 4;
                const int mh = m / 128, mm = m % 128;
                const int c  = mm / 8;
                // k group of K step 0, first half: kg = 2*(b/2); other (kk, h) add
                // (kk*4 + h) * MH * 1024 bytes and leave (kg >> 1) & 1 == b/2
                frag_off[i] = ((2 * (b / 2)) * MH + mh) * 1024
                              + (j * 16 + (c ^ (4 * j) ^ (2 * (b / 2)))) * 16 + (mm % 8) * 2;
            }
        }
        else
        {
            // 16-lane block g reads k = 8g + 4h + j (h: which of the two reads), rows
            // 16i .. 16i+15 of the wave tile: kg = kk*8 + 2g + h, (kg >> 1) & 1 == g & 1
            const int g = lane / 16, s = lane % 16, j = s / 4;
#pragma unroll
            for(int i = 0; i < T; ++i)
            {
                const int m  = wave_row0 + i * 16 + (s % 4) * 4;
                const int mh = m / 128, mm = m % 128;
                const int c  = mm / 8;
                frag_off[i] = ((2 * g) * MH + mh) * 1024
                              + (j * 16 + (c ^ (4 * j) ^ (2 * (g & 1)))) * 16 + (mm % 8) * 2;
            }
        }
    }

    // Enqueue this wave's share of one tile: global (tile_origin + lane_off) -> LDS.
    template<class InT>
    __device__ __forceinline__ void issue(const InT* tile_origin, lds_char_ptr lds_tile, int wave) const
    {
#pragma unroll
        for(int i = 0; i < PER_WAVE; ++i)
        {
            const int t = wave + i * WAVES;
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void*)(tile_origin + lane_off[i]),
                (__attribute__((address_space(3))) void*)(lds_tile + t * 1024),
                16,
                0,
                RWG_LOAD_AUX);
        }
    }

    // fragment() as volatile inline assembly, for the hand-scheduled kernel: the reads
    // stay where the source puts them and the compiler neither tracks them (the caller
    // waits with s_waitcnt lgkmcnt before the first use) nor orders them against the
    // global -> LDS loads (behind such a load it puts s_waitcnt vmcnt(0) in front of
    // every ds_read_b64_tr_b16 it knows of).  lds_tile is the byte address of the
    // operand tile in LDS.
    template<int I, int KKI>
    __device__ __forceinline__ u32x4 fragment_pinned(unsigned int lds_tile) const
    {
        if constexpr(KMAJOR)
        {
            u32x4              r;
            const unsigned int addr = lds_tile + (unsigned int)frag_off[KKI];
            asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(I * (MI * 16 * CH)));
            return r;
        }
        else
        {
            uint2              lo, hi;
            const unsigned int addr = lds_tile + (unsigned int)frag_off[I];
            asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2"
                         : "=v"(lo)
                         : "v"(addr), "n"((KKI * (KSTEP / 4) + 0) * MH * 1024));
            asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2"
                         : "=v"(hi)
                         : "v"(addr), "n"((KKI * (KSTEP / 4) + 1) * MH * 1024));
            return u32x4{lo.x, lo.y, hi.x, hi.y};
        }
    }

    // MFMA operand registers of operand tile i for K step kk.
    __device__ __forceinline__ u32x4 fragment(lds_char_ptr lds_tile, int i, int kk) const
    {
        if constexpr(KMAJOR)
        {
            return *reinterpret_cast<__attribute__((address_space(3))) u32x4*>(
                lds_tile + frag_off[kk] + i * (MI * 16 * CH));
        }
        else
        {
            auto* p0 = reinterpret_cast<__attribute__((address_space(3))) fp16x4_raw*>(
                lds_tile + frag_off[i] + (kk * (KSTEP / 4) + 0) * MH * 1024);
            auto* p1 = reinterpret_cast<__attribute__((address_space(3))) fp16x4_raw*>(
                lds_tile + frag_off[i] + (kk * (KSTEP / 4) + 1) * MH * 1024);
            const fp16x4_raw lo = __builtin_amdgcn_ds_read_tr16_b64_v4f16(p0);
            const fp16x4_raw hi = __builtin_amdgcn_ds_read_tr16_b64_v4f16(p1);
            const uint2      l2 = __builtin_bit_cast(uint2, lo);
            const uint2      h2 = __builtin_bit_cast(uint2, hi);
            return u32x4{l2.x, l2.y, h2.x, h2.y};
        }
    }
};

// Accumulator registers of one MFMA tile: 32x32 -> 16 per lane, 16x16 -> 4.
template<int MI>
using mfma_acc = typename std::conditional<MI == 32, f32x16, f32x4>::type;

// acc += A-fragment x B-fragment for one MI x MI tile of C.  With the 16x16x32 shape
// the operands go in swapped: the MFMA then computes the transposed tile, and a lane
// ends up with 4 consecutive columns of one row of C.
template<in_kind IN, int MI>
__device__ __forceinline__ mfma_acc<MI> mfma_tile(u32x4 fa, u32x4 fb, mfma_acc<MI> acc)
{
    if constexpr(MI == 32)
    {
        return mfma_32x32x16<IN>(fa, fb, acc);
    }
    else
    {
        return mfma_16x16x32<IN>(fb, fa, acc);
    }
}

// Store this wave's accumulators to a row-major M x N matrix of DstT (C itself, or
// fp32 split-K partial sums) whose rows are `pitch` elements apart and whose wave tile
// starts at (row_w, col_w); M and N bound the guarded stores.
template<int MI, bool GUARD_C, int TM, int TN, class AccT, class DstT>
__device__ __forceinline__ void write_out(const AccT (&acc)[TM][TN],
                                          DstT*     D,
                                          int       M,
                                          int       N,
                                          long long pitch,
                                          int       row_w,
                                          int       col_w,
                                          int       lane)
{
    if constexpr(MI == 32)
    {
        // Accumulator register v of a 32x32 tile is row 8*(v/4) + 4*(lane/32) + v%4,
        // column lane%32.
        const int lane_lo = lane & 31, lane_hi = lane >> 5;
#pragma unroll
        for(int i = 0; i < TM; ++i)
        {
#pragma unroll
            for(int j = 0; j < TN; ++j)
            {
                const int col = col_w + j * 32 + lane_lo;
#pragma unroll
                for(int v = 0; v < 16; ++v)
                {
                    const int row = row_w + i * 32 + 8 * (v / 4) + 4 * lane_hi + (v % 4);
                    if(!GUARD_C || (row < M && col < N))
                    {
                        D[(long long)row * pitch + col] = to_out<DstT>(acc[i][j][v]);
                    }
                }
            }
        }
    }
    else
    {
        // Transposed 16x16 tiles (the kernels feed the MFMA with B's fragment first): register v of tile (i, j) is row
        // lane%16 of the tile, column 4*(lane/16) + v.  Whole tiles with an aligned
        // destination take one 8- or 16-byte store per tile and lane.
        const int r16 = lane & 15, g = lane >> 4;
#pragma unroll
        for(int i = 0; i < TM; ++i)
        {
            const int row = row_w + i * 16 + r16;
#pragma unroll
            for(int j = 0; j < TN; ++j)
            {
                const int       col = col_w + j * 16 + 4 * g;
                const long long at  = (long long)row * pitch + col;
                if constexpr(GUARD_C)
                {
#pragma unroll
                    for(int v = 0; v < 4; ++v)
                    {
                        if(row < M && col + v < N)
                        {
                            D[at + v] = to_out<DstT>(acc[i][j][v]);
                        }
                    }
                }
                else
                {
                    typedef DstT dst4 __attribute__((ext_vector_type(4)));
                    dst4 o;
#pragma unroll
                    for(int v = 0; v < 4; ++v)
                    {
                        o[v] = to_out<DstT>(acc[i][j][v]);
                    }
                    *reinterpret_cast<dst4*>(D + at) = o;
                }
            }
        }
    }
}

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
struct direct_gemm
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
    static_assert(STAGES == 2 || STAGES == 4, "stage ring must be a power of two");
    static_assert(KK % 2 == 0, "operand double-buffer parity must repeat every tile");
    static_assert(LDS_BYTES <= 160 * 1024, "tile ring does not fit the 160 KB LDS");

    using op_a = direct_operand<A_KMAJOR, BM, BK, WTM, WAVES, MI>;
    using op_b = direct_operand<B_KMAJOR, BN, BK, WTN, WAVES, MI>;
    using acc_t = mfma_acc<MI>;
    static constexpr int ACC_REGS = MI == 32 ? 16 : 4;

    static constexpr int VM_LOADS = op_a::PER_WAVE + op_b::PER_WAVE; // per wave, per tile
    static constexpr int DS_READS = TM * op_a::DS_PER_FRAGMENT + TN * op_b::DS_PER_FRAGMENT;
    static_assert((STAGES - 1) * VM_LOADS < 64, "vmcnt is a 6-bit counter");

    // s_waitcnt immediate: lgkmcnt(0), expcnt untouched, vmcnt(n)
    static constexpr int waitcnt_imm(int vmcnt)
    {
        return (vmcnt & 15) | (7 << 4) | (0 << 8) | ((vmcnt >> 4) << 14);
    }

    // With an operand that is contiguous along M or N the fragment reads are volatile
    // inline assembly: behind a global -> LDS load the compiler puts s_waitcnt vmcnt(0) in
    // front of every ds_read_b64_tr_b16 it knows of, which waits for the loads of the
    // tiles further down the ring too and leaves the ring one tile deep in effect (at
    // 2048^3 the M/N-contiguous layouts ran 20-30 % behind the K-contiguous one, more
    // with a ring of 4).  The compiler does not track these reads, so each call first
    // waits for the reads of the call before it, whose fragments the MFMAs that follow
    // this call consume, and the caller waits once more behind the K loop.
    static constexpr bool PINNED_READS = !A_KMAJOR || !B_KMAJOR;

    template<int KKI, int... I, int... J>
    __device__ __forceinline__ static void read_pinned(std::integer_sequence<int, I...>,
                                                       std::integer_sequence<int, J...>,
                                                       const op_a&  oa,
                                                       const op_b&  ob,
                                                       unsigned int stage,
                                                       u32x4 (&fa)[TM],
                                                       u32x4 (&fb)[TN])
    {
        ((fa[I] = oa.template fragment_pinned<I, KKI>(stage)), ...);
        ((fb[J] = ob.template fragment_pinned<J, KKI>(stage + A_BYTES)), ...);
    }

    __device__ __forceinline__ static void load_fragments(const op_a& oa,
                                                          const op_b& ob,
                                                          lds_char_ptr stage,
                                                          int          kk,
                                                          u32x4 (&fa)[TM],
                                                          u32x4 (&fb)[TN])
    {
        if constexpr(PINNED_READS)
        {
            static_assert(KK <= 4, "one case per K step below");
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_sched_barrier(0); // no MFMA of this phase in front of the wait
            const unsigned int addr = (unsigned int)(size_t)stage;
            constexpr auto     sa = std::make_integer_sequence<int, TM>{};
            constexpr auto     sb = std::make_integer_sequence<int, TN>{};
            // kk is a constant after unrolling
            if(kk == 0)
            {
                read_pinned<0>(sa, sb, oa, ob, addr, fa, fb);
            }
            else if(kk == 1)
            {
                read_pinned<1 % KK>(sa, sb, oa, ob, addr, fa, fb);
            }
            else if(kk == 2)
            {
                read_pinned<2 % KK>(sa, sb, oa, ob, addr, fa, fb);
            }
            else
            {
                read_pinned<3 % KK>(sa, sb, oa, ob, addr, fa, fb);
            }
        }
        else
        {
#pragma unroll
            for(int i = 0; i < TM; ++i)
            {
                fa[i] = oa.fragment(stage, i, kk);
            }
#pragma unroll
            for(int j = 0; j < TN; ++j)
            {
                fb[j] = ob.fragment(stage + A_BYTES, j, kk);
            }
        }
    }

    __device__ __forceinline__ static void
        multiply(const u32x4 (&fa)[TM], const u32x4 (&fb)[TN], acc_t (&acc)[TM][TN])
    {
#pragma unroll
        for(int i = 0; i < TM; ++i)
        {
#pragma unroll
            for(int j = 0; j < TN; ++j)
            {
                acc[i][j] = mfma_tile<IN, MI>(fa[i], fb[j], acc[i][j]);
            }
        }
    }

    // Ask the scheduler for "one MFMA, then a slice of the memory instructions" so
    // the LDS reads and global loads of a phase ride under its MFMAs instead of
    // running ahead of or behind them.  LDS reads go under the first MFMAs, global
    // -> LDS loads under the rest (they follow the reads in program order: the
    // compiler keeps LDS reads and LDS-writing loads in source order).
    template<int N_DS, int N_VMEM>
    __device__ __forceinline__ static void interleave_hint()
    {
        constexpr int MFMAS    = TM * TN;
        constexpr int DS_SLOTS = N_DS == 0 ? 0 : (N_VMEM > 0 ? MFMAS / 2 : MFMAS);
        constexpr int DS_PER   = DS_SLOTS > 0 ? (N_DS + DS_SLOTS - 1) / DS_SLOTS : 1;
        constexpr int VM_SLOTS = N_VMEM == 0 ? 0 : MFMAS - DS_SLOTS;
        constexpr int VM_PER   = VM_SLOTS > 0 ? (N_VMEM + VM_SLOTS - 1) / VM_SLOTS : 1;
        constexpr int REST     = MFMAS - DS_SLOTS - VM_SLOTS;
#pragma unroll
        for(int d = 0; d < DS_SLOTS; ++d)
        {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); // 1 MFMA
            if(d * DS_PER < N_DS)
            {
                __builtin_amdgcn_sched_group_barrier(0x100, DS_PER, 0); // LDS reads
            }
        }
        // loads are spread evenly: every VM_GAP-th MFMA slot carries VM_PER of them
        constexpr int VM_GAP = (N_VMEM > 0 && VM_SLOTS >= 2 * N_VMEM) ? VM_SLOTS / N_VMEM : 1;
#pragma unroll
        for(int v = 0; v < VM_SLOTS; ++v)
        {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if(v % VM_GAP == 0 && (v / VM_GAP) * VM_PER < N_VMEM)
            {
                __builtin_amdgcn_sched_group_barrier(0x020, VM_PER, 0); // global -> LDS
            }
        }
        if constexpr(REST > 0)
        {
            __builtin_amdgcn_sched_group_barrier(0x008, REST, 0);
        }
    }

    // One BK-wide tile out of stage (it % STAGES).  Every tile runs the same
    // straight-line code, so that the scheduler can interleave it and no register
    // shuffling is needed between variants of the step:
    //   * (4-deep ring only) before the barrier, operand B of tile it+STAGES-1 is
    //     enqueued; its operand A went out after the previous tile's barrier;
    //   * after the barrier, tile it+STAGES is enqueued into the stage just drained
    //     (2-deep ring: both operands; 4-deep ring: operand A only);
    //   * K step 0 of tile it+1 is pre-read under the last K step's MFMAs.
    // Past the end of K the caller keeps the source pointers on the last tile: the
    // redundant loads land in stages nobody reads again, and the pre-read values are
    // never used.  That keeps the number of loads in flight behind tile it+1 a
    // compile-time constant, which s_waitcnt needs.
    // Splitting a tile's loads over two phases keeps the rate at which the waves
    // hand loads to the texture addresser (16 cycles per 1 KiB load, one addresser
    // per CU) below what it drains, so MFMA issue does not stall behind them.
    static constexpr bool SPLIT_ISSUE = STAGES == 4;
    static constexpr int  WAIT_VM     = (STAGES - 2) * VM_LOADS;

    __device__ __forceinline__ static void tile_step(const op_a&  oa,
                                                     const op_b&  ob,
                                                     lds_char_ptr lds,
                                                     int          it,
                                                     int          wave,
                                                     const InT*   a_src,
                                                     const InT*   b_src,
                                                     u32x4 (&fa)[2][TM],
                                                     u32x4 (&fb)[2][TN],
                                                     acc_t (&acc)[TM][TN])
    {
        lds_char_ptr cur = lds + (it & (STAGES - 1)) * STAGE;
        lds_char_ptr nxt = lds + ((it + 1) & (STAGES - 1)) * STAGE;
#pragma unroll
        for(int kk = 0; kk + 1 < KK; ++kk)
        {
            const int use = kk & 1, fill = use ^ 1;
            load_fragments(oa, ob, cur, kk + 1, fa[fill], fb[fill]);
            if constexpr(SPLIT_ISSUE)
            {
                if(kk == 0)
                {
                    ob.issue(b_src, lds + ((it + STAGES - 1) & (STAGES - 1)) * STAGE + A_BYTES, wave);
                }
            }
            multiply(fa[use], fb[use], acc);
            if(SPLIT_ISSUE && kk == 0)
            {
                interleave_hint<DS_READS, op_b::PER_WAVE>();
            }
            else
            {
                interleave_hint<DS_READS, 0>();
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // Every read of `cur` has been issued; once they have landed and this wave's
        // share of tile it+1 is in LDS, meet the other waves.  After the barrier
        // `cur` may be overwritten and `nxt` may be read.
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(WAIT_VM));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        constexpr int use = (KK - 1) & 1, fill = use ^ 1;
        load_fragments(oa, ob, nxt, 0, fa[fill], fb[fill]);
        oa.issue(a_src, cur, wave);
        if constexpr(!SPLIT_ISSUE)
        {
            ob.issue(b_src, cur + A_BYTES, wave);
        }
        multiply(fa[use], fb[use], acc);
        interleave_hint<DS_READS, SPLIT_ISSUE ? op_a::PER_WAVE : VM_LOADS>();
        __builtin_amdgcn_sched_barrier(0);
    }

    __device__ __forceinline__ static void run(const gemm_args& args)
    {
        __shared__ __attribute__((aligned(1024))) char lds_raw[LDS_BYTES];
        lds_char_ptr lds = (lds_char_ptr)lds_raw;

        const int tid     = threadIdx.x;
        const int lane    = tid & 63;
        const int wave    = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int wave_m  = wave / WAVES_N;
        const int wave_n  = wave % WAVES_N;

        // The hardware deals the workgroups of the grid, x fastest, round-robin over the
        // XCDs.  With batch_by_xcd (whole tiles only) each XCD takes a contiguous run of
        // (batch entry, tile) pairs instead of every eighth tile of every entry.
        block_work w;
        tile_coord t;
        long long  batch;
        if(args.batch_by_xcd)
        {
            const int item = xcd_remap((int)(blockIdx.x + blockIdx.y * gridDim.x), (int)(gridDim.x * gridDim.y));
            const int entry = item / (int)gridDim.x;
            batch           = entry;
            w               = decode_block(args, item - entry * (int)gridDim.x);
            t = banded_tile(w.tile_id, args.grid_m, args.grid_n, args.group);
        }
        else
        {
            batch = blockIdx.y;
            w     = decode_block(args);
            t     = map_tile(w.tile_id, args.grid_m, args.grid_n, args.group);
        }
        const int slice = w.slice;
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

        // tile origins at this slice's first K step; advanced by BK per tile
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
                for(int v = 0; v < ACC_REGS; ++v)
                {
                    acc[i][j][v] = 0.0f;
                }
            }
        }

        if(nk > 0)
        {
            u32x4 fa[2][TM], fb[2][TN];

            // Source pointers never move past the last tile of this K range.
            const InT* a_last = a_src + (long long)(nk - 1) * a_step;
            const InT* b_last = b_src + (long long)(nk - 1) * b_step;

            // Prologue: fill the ring and wait for tile 0.  The 2-deep ring takes tiles
            // 0 and 1 whole; the 4-deep ring takes tiles 0..2 whole and operand A of
            // tile 3, whose operand B goes out during tile 0.
#pragma unroll
            for(int s = 0; s < STAGES; ++s)
            {
                oa.issue(a_src, lds + s * STAGE, wave);
                a_src = a_src + a_step > a_last ? a_last : a_src + a_step;
                if(!(SPLIT_ISSUE && s == STAGES - 1))
                {
                    ob.issue(b_src, lds + s * STAGE + A_BYTES, wave);
                    b_src = b_src + b_step > b_last ? b_last : b_src + b_step;
                }
            }
            __builtin_amdgcn_s_waitcnt(
                waitcnt_imm((STAGES - 1) * VM_LOADS - (SPLIT_ISSUE ? op_b::PER_WAVE : 0)));
            __builtin_amdgcn_s_barrier();
            load_fragments(oa, ob, lds, 0, fa[0], fb[0]);

            for(int it = 0; it < nk; ++it)
            {
                tile_step(oa, ob, lds, it, wave, a_src, b_src, fa, fb, acc);
                a_src = a_src + a_step > a_last ? a_last : a_src + a_step;
                b_src = b_src + b_step > b_last ? b_last : b_src + b_step;
            }
            // redundant tail loads, and the last fragment reads (nobody uses them, but they
            // must not land in registers that hold something else by then), may still be
            // in flight
            __builtin_amdgcn_s_waitcnt(waitcnt_imm(0));
            __builtin_amdgcn_sched_barrier(0);
        }

        if(w.slices == 1)
        {
            OutT* C = static_cast<OutT*>(args.C) + batch * args.batch_stride_c;
            write_out<MI, GUARD_C>(acc, C, args.M, args.N, args.N, row0 + wave_m * WTM, col0 + wave_n * WTN, lane);
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

#endif // ROCM_WMMA_GEMM_DIRECT_KERNEL_HPP
