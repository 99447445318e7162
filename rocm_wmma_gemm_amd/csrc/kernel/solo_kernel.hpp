// One-wave-per-SIMD MFMA GEMM kernel for gfx950 (4 waves, 128 x 128 wave tiles; also
// 96-wide ones), with persistent workgroups.
//
// Same LDS layouts as the direct kernel (direct_kernel.hpp: swizzled K-contiguous rows,
// ds_read_b64_tr_b16 for operands that are contiguous along M or N) on the 16x16x32
// MFMA, but with the largest wave tile the register file allows: 128 x 128 per wave =
// 256 accumulator registers, all of the AGPRs.  A wave then reads 16 operand fragments
// from LDS per 64 MFMAs, against 12 per 32 for the 128 x 64 wave tiles of the 8-wave
// kernels: one third fewer LDS bytes per FLOP, which is what the power-capped clock
// responds to.
//
// With one wave per SIMD nothing hides a stall, so the schedule is fixed by hand:
// the MFMAs are volatile inline assembly (which also pins every accumulator to its
// AGPRs: with the builtin the register allocator moved accumulators between the two
// register files inside the loop), and the LDS reads and global -> LDS loads (buffer
// loads, also inline assembly) of a K step sit between them in source order.
//
// Ring of 2 tiles of BLOCK_K 64 (two MFMA K steps per tile, one barrier per tile;
// K-contiguous rows are 128 bytes, so every load fetches whole cache lines).  The
// fragments of the next K step are always read one step ahead, so the stage of the
// tile being multiplied is free for the next loads as soon as all waves have passed
// the barrier in the middle of the tile.  Measured with the shader clock on 8192^3:
// 1117 + 1186 cycles for the two steps of a tile (1024 each would be MFMA-bound) plus
// about 70 in the wait and the barrier, where issuing a tile's loads back to back
// had cost 1700-1900 cycles for the second step.
//
// The same kernel with BLOCK_K 32 keeps a ring of 4 tiles of one MFMA K step each (the
// same 128 KB of LDS): a barrier per K step, and the loads of tile t+4 go out under tile
// t, so a load has two to three tile times to land instead of a quarter to one.  Built to
// see whether the fall of the rate for K-contiguous operands that no longer fit the 256 MB
// memory-side cache (8192 x 8192 x 28672: 1250 TFLOP/s against 1540 at K = 8192) is a
// matter of load latency.  It is not: the ring of 4 runs 1236 there, and 5..13 % below the
// ring of 2 where the operands stay in that cache (the second barrier, and the 64-byte
// half lines a K-contiguous row of 32 fetches).  What the counters show instead for those
// shapes is the texture addresser stalled by the L1 four times as often as in the vendor's
// kernel of the same tile, and L2 misses that take 850 cycles against 620.
//
// A launch has one workgroup per CU; each works through its tiles (or K slices, or a
// range of K tiles: see walk) with one load stream running through all of them, and
// stores C through per-wave LDS strips as 16-byte buffer stores.  Loads and stores go
// through buffer descriptors whose range check handles the ragged edges of a matrix.
//
// Role with respect to the reference: as the other kernels, its gemm_impl (reference
// rocm_wmma_gemm/include/rocm_wmma_gemm/kernel/kernel.hpp:108-556).
#ifndef ROCM_WMMA_GEMM_SOLO_KERNEL_HPP
#define ROCM_WMMA_GEMM_SOLO_KERNEL_HPP

#include <utility>

#include "direct_kernel.hpp"

// Schedule constants of the K loop, as macros so that the tuner's run-time compile
// (kernel_jit.hip) can try others: a fragment read after every RWG_SOLO_FRAG_GAP-th MFMA;
// RWG_SOLO_LATE_LOADS_16THS sixteenths of a tile's loads issued in the first step of the next
// tile (one every RWG_SOLO_LATE_GAP MFMAs), the rest under the second step of this one.
#ifndef RWG_SOLO_FRAG_GAP
#define RWG_SOLO_FRAG_GAP 2
#endif
#ifndef RWG_SOLO_LATE_LOADS_16THS
#define RWG_SOLO_LATE_LOADS_16THS 4
#endif
#ifndef RWG_SOLO_LATE_GAP
#define RWG_SOLO_LATE_GAP 4
#endif

namespace rocm_wmma_gemm
{
namespace device
{

// acc += (B fragment) x (A fragment): the transposed 16x16 tile, see write_out.
template<in_kind IN>
__device__ __forceinline__ void mfma_16x16x32_pinned(f32x4& acc, const u32x4& fa, const u32x4& fb)
{
    if constexpr(IN == in_kind::f16)
    {
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(fb), "v"(fa));
    }
    else
    {
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(fb), "v"(fa));
    }
}

// K_RUNS: the twin that walks an item's K tiles in runs and groups (run(), below).
// ONCE (twin only): bit 0, the K-loop loads of B carry the non-temporal hint, bit 1, those of
// A.  For an operand of 256 MB and more that a single row (column) of tiles reads, so that
// every line of it is wanted exactly once: it cannot stay in the memory-side cache for
// anybody, and without the hint its lines push out the small operand's and the partial sums'.
// bf16, 256 rows against 28672 x 8192 weights through the tuned plans: 820 -> 908 TFLOP/s
// with B column-major, 836 -> 860 row-major, fp32 out 802 -> 908 with everything
// column-major.  With two to four rows of tiles the hint is worth +6..15 % on the plain walk
// but loses 2..14 % with the K order, whose point is that the second sharer finds the line
// in L2 (hinted lines are the first to go), and with 32 rows of tiles, where the panels are
// shared between XCDs through the memory-side cache, it costs 15 %: the host sets it by shape.
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
         bool K_RUNS  = false,
         int  ONCE    = 0>
struct solo_gemm
{
    using InT = typename std::conditional<IN == in_kind::f16, _Float16, __bf16>::type;

    static constexpr int MI        = 16;
    static constexpr int WAVES     = WAVES_M * WAVES_N;
    static constexpr int THREADS   = 64 * WAVES;
    static constexpr int WTM       = BM / WAVES_M;
    static constexpr int WTN       = BN / WAVES_N;
    static constexpr int TM        = WTM / MI;
    static constexpr int TN        = WTN / MI;
    static constexpr int MFMAS     = TM * TN;
    static constexpr int A_BYTES   = BM * BK * 2;
    static constexpr int B_BYTES   = BN * BK * 2;
    static constexpr int STAGE     = A_BYTES + B_BYTES;
    static constexpr int LDS_BYTES = STAGES * STAGE;
    static_assert((BK == 64 && STAGES == 2) || (BK == 32 && STAGES == 4),
                  "ring of 2 tiles of BLOCK_K 64, or of 4 tiles of BLOCK_K 32");

    using op_a = direct_operand<A_KMAJOR, BM, BK, WTM, WAVES, MI>;
    using op_b = direct_operand<B_KMAJOR, BN, BK, WTN, WAVES, MI>;

    static constexpr int VM_LOADS = op_a::PER_WAVE + op_b::PER_WAVE; // per wave, per tile
    static_assert((STAGES - 1) * VM_LOADS < 64, "vmcnt is a 6-bit counter");

    static constexpr int KK    = BK / 32; // MFMA K steps per tile
    static constexpr int FRAGS = TM + TN;
    // Fragment u (A fragments first, then B) is read after MFMA u * FRAG_GAP.
    static constexpr int FRAG_GAP = RWG_SOLO_FRAG_GAP;
    static_assert(FRAGS * FRAG_GAP <= MFMAS, "fragment reads must fit under the MFMAs of a step");

    // s_waitcnt immediate: lgkmcnt(0), expcnt untouched, vmcnt(n)
    static constexpr int waitcnt_imm(int vmcnt)
    {
        return (vmcnt & 15) | (7 << 4) | (0 << 8) | ((vmcnt >> 4) << 14);
    }

    // Largest range a load descriptor is given; a vector offset of this value is outside
    // every descriptor's range, whatever the scalar offset adds (tile spans stay below it,
    // so the sum does not wrap).
    static constexpr unsigned int RANGE_MAX = 0x80000000u;

    // Addressing of one operand's global -> LDS loads.  Load i of a tile (i = 0 ..
    // PER_WAVE-1; it fills the 1 KiB LDS block wave + i*WAVES) is a buffer load whose
    // address is split three ways so that nothing is computed per load: the tile origin
    // sits in the buffer descriptor (scalar registers, advanced once per tile), the
    // part that depends on i is a scalar offset i * stride, and the lane's own part is
    // a vector offset that is the same for every i (K-contiguous: the swizzle of row
    // RPL*(wave + 4i) + lane/CH does not depend on i) or alternates between two values
    // with the parity of i (M/N-contiguous: the swizzle term 2*((kg/2)%2) does).
    template<bool KMAJOR, int ROWS>
    struct load_addr
    {
        static_assert(WAVES == 4 && (KMAJOR || ROWS == 256), "derived for this tile and wave count");
        static constexpr int CH  = BK / 8; // 16-byte chunks of a K-contiguous row
        static constexpr int RPL = 64 / CH; // rows of it that one load fills
        unsigned int voff[KMAJOR ? 1 : 2]; // bytes
        unsigned int stride; // bytes between load i and load i+1

        __device__ __forceinline__ void init(int wave, int lane, long long ld)
        {
            if constexpr(KMAJOR)
            {
                const int r = RPL * wave + lane / CH; // row of load 0; load i adds WAVES * RPL rows
                const int c = (lane % CH) ^ swizzle_of_row<CH, MI>(r);
                voff[0]     = (unsigned int)((r * ld + c * 8) * 2);
                stride      = (unsigned int)(WAVES * RPL * ld * 2);
            }
            else
            {
                // block t = wave + 4i: k group kg = t/2 = wave/2 + 2i, 128-row half mh = wave%2
                const int j = lane / 16, cphys = lane % 16;
#pragma unroll
                for(int p = 0; p < 2; ++p) // p = (kg/2) % 2 = i % 2
                {
                    const int c = cphys ^ (4 * j) ^ (2 * p);
                    voff[p]     = (unsigned int)((((wave >> 1) * 4 + j) * ld + (wave & 1) * 128 + c * 8) * 2);
                }
                stride = (unsigned int)(8 * ld * 2);
            }
        }

        template<int I>
        __device__ __forceinline__ unsigned int vector_offset() const
        {
            return voff[KMAJOR ? 0 : (I & 1)];
        }

        // The offsets for a last K tile of which only columns [0, kt) exist, kt a multiple
        // of 8.  K-contiguous: a lane fetches the same 8 columns of its row in every load,
        // and a lane whose columns lie past kt gets an offset outside every descriptor's
        // range (RANGE_MAX), so its loads write zeros to LDS.  M/N-contiguous: the rows
        // past kt lie past the end of the operand's batch entry, where the descriptor
        // ends; nothing to change.
        __device__ __forceinline__ load_addr for_tail(int lane, int wave, int kt) const
        {
            load_addr t = *this;
            if constexpr(KMAJOR)
            {
                const int r = RPL * wave + lane / CH;
                const int c = (lane % CH) ^ swizzle_of_row<CH, MI>(r);
                t.voff[0]   = c * 8 < kt ? voff[0] : RANGE_MAX;
            }
            return t;
        }

        // this, or other when `take` (the same in every lane) is set
        __device__ __forceinline__ load_addr or_else(bool take, const load_addr& other) const
        {
            load_addr t = *this;
#pragma unroll
            for(int p = 0; p < (KMAJOR ? 1 : 2); ++p)
            {
                t.voff[p] = take ? other.voff[p] : voff[p];
            }
            return t;
        }
    };

    using addr_a = load_addr<A_KMAJOR, BM>;
    using addr_b = load_addr<B_KMAJOR, BN>;

    // The same pointer, held in scalar registers (it must be the same in every lane).
    __device__ __forceinline__ static const InT* scalar_pointer(const InT* p)
    {
        const unsigned long long v  = (unsigned long long)p;
        const unsigned int       lo = __builtin_amdgcn_readfirstlane((unsigned int)v);
        const unsigned int       hi = __builtin_amdgcn_readfirstlane((unsigned int)(v >> 32));
        return (const InT*)(((unsigned long long)hi << 32) | lo);
    }

    // 128-bit buffer descriptor of a tile: base = its origin, no stride, raw 32-bit format,
    // and a range that ends where the operand's allocation ends (`end`), so that a tile
    // that hangs over the edge of a ragged matrix cannot read past it: a load beyond the
    // range, whether through the vector or the scalar offset, writes zeros to LDS
    // (mfma_probe --range).  Rows or columns past the edge but inside the allocation
    // read whatever is there (the next k row, the next batch entry); they only reach
    // accumulators of rows and columns of C that the guarded stores leave out.  Every
    // tile span fits 31 bits (the host checks).
    __device__ __forceinline__ static u32x4 descriptor(const InT* origin, const InT* end)
    {
        const unsigned long long p = (unsigned long long)origin;
        unsigned int             records = 0xffffffffu;
        if constexpr(GUARD_C)
        {
            // (whole tiles of a matrix of whole tiles end inside it anyway)
            const unsigned long long left = (unsigned long long)end - p;
            records                       = left > RANGE_MAX ? RANGE_MAX : (unsigned int)left;
        }
        return u32x4{(unsigned int)p, (unsigned int)(p >> 32) & 0xffffu, records, 0x00020000u};
    }

    // One MFMA and, in its shadow, one global -> LDS load: M0 (the load's LDS
    // destination) is written before the MFMA, which fills the wait state M0 needs
    // before the load may use it.  lds_block = LDS byte address of this wave's block 0
    // of the operand's stage; LDS_IMM = i * WAVES * 1024.
    // NT: the load carries the non-temporal hint (ONCE, below).
    template<int LDS_IMM, bool NT = false>
    __device__ __forceinline__ static void mfma_and_load(f32x4&       acc,
                                                         const u32x4& fa,
                                                         const u32x4& fb,
                                                         unsigned int lds_block,
                                                         unsigned int voff,
                                                         const u32x4& rsrc,
                                                         unsigned int soff)
    {
        if constexpr(NT)
        {
            if constexpr(IN == in_kind::f16)
            {
                asm volatile("s_add_u32 m0, %[ldsb], %[imm]\n\t"
                             "v_mfma_f32_16x16x32_f16 %[acc], %[b], %[a], %[acc]\n\t"
                             "buffer_load_dwordx4 %[voff], %[rsrc], %[soff] offen nt lds"
                             : [acc] "+a"(acc)
                             : [b] "v"(fb), [a] "v"(fa), [ldsb] "s"(lds_block), [imm] "n"(LDS_IMM),
                               [voff] "v"(voff), [rsrc] "s"(rsrc), [soff] "s"(soff)
                             : "memory", "scc");
            }
            else
            {
                asm volatile("s_add_u32 m0, %[ldsb], %[imm]\n\t"
                             "v_mfma_f32_16x16x32_bf16 %[acc], %[b], %[a], %[acc]\n\t"
                             "buffer_load_dwordx4 %[voff], %[rsrc], %[soff] offen nt lds"
                             : [acc] "+a"(acc)
                             : [b] "v"(fb), [a] "v"(fa), [ldsb] "s"(lds_block), [imm] "n"(LDS_IMM),
                               [voff] "v"(voff), [rsrc] "s"(rsrc), [soff] "s"(soff)
                             : "memory", "scc");
            }
        }
        else
        {
            if constexpr(IN == in_kind::f16)
            {
                asm volatile("s_add_u32 m0, %[ldsb], %[imm]\n\t"
                             "v_mfma_f32_16x16x32_f16 %[acc], %[b], %[a], %[acc]\n\t"
                             "buffer_load_dwordx4 %[voff], %[rsrc], %[soff] offen lds"
                             : [acc] "+a"(acc)
                             : [b] "v"(fb), [a] "v"(fa), [ldsb] "s"(lds_block), [imm] "n"(LDS_IMM),
                               [voff] "v"(voff), [rsrc] "s"(rsrc), [soff] "s"(soff)
                             : "memory", "scc");
            }
            else
            {
                asm volatile("s_add_u32 m0, %[ldsb], %[imm]\n\t"
                             "v_mfma_f32_16x16x32_bf16 %[acc], %[b], %[a], %[acc]\n\t"
                             "buffer_load_dwordx4 %[voff], %[rsrc], %[soff] offen lds"
                             : [acc] "+a"(acc)
                             : [b] "v"(fb), [a] "v"(fa), [ldsb] "s"(lds_block), [imm] "n"(LDS_IMM),
                               [voff] "v"(voff), [rsrc] "s"(rsrc), [soff] "s"(soff)
                             : "memory", "scc");
            }
        }
    }

    // A load on its own (prologue).
    template<int LDS_IMM>
    __device__ __forceinline__ static void load_only(unsigned int lds_block,
                                                     unsigned int voff,
                                                     const u32x4& rsrc,
                                                     unsigned int soff)
    {
        // (the compiler does not look for hazards around inline assembly: four wait
        // states cover a descriptor or offset that a v_readfirstlane has just written)
        asm volatile("s_add_u32 m0, %[ldsb], %[imm]\n\t"
                     "s_nop 4\n\t"
                     "buffer_load_dwordx4 %[voff], %[rsrc], %[soff] offen lds"
                     :
                     : [ldsb] "s"(lds_block), [imm] "n"(LDS_IMM), [voff] "v"(voff), [rsrc] "s"(rsrc),
                       [soff] "s"(soff)
                     : "memory", "scc");
    }

    // One dword per lane from 64 different cache lines, fetched for the sake of the fetch:
    // the lines travel from memory into this XCD's L2 (and the dwords into 256 bytes of LDS
    // that nothing reads).  Its range ends with the operand's allocation, so a touch past
    // the end of a matrix fetches nothing.
    __device__ __forceinline__ static void touch_lines(unsigned int lds_sink, unsigned int voff,
                                                       const InT* origin, const InT* end, unsigned int soff)
    {
        const unsigned long long p    = (unsigned long long)origin;
        const unsigned long long left = (unsigned long long)end > p ? (unsigned long long)end - p : 0;
        const u32x4 rsrc{(unsigned int)p, (unsigned int)(p >> 32) & 0xffffu,
                         left > RANGE_MAX ? RANGE_MAX : (unsigned int)left, 0x00020000u};
        asm volatile("s_mov_b32 m0, %[sink]\n\t"
                     "s_nop 4\n\t"
                     "buffer_load_dword %[voff], %[rsrc], %[soff] offen lds"
                     :
                     : [sink] "s"(lds_sink), [voff] "v"(voff), [rsrc] "s"(rsrc), [soff] "s"(soff)
                     : "memory");
    }

    // Everything a step works on.
    struct step_ctx
    {
        const op_a&   oa;
        const op_b&   ob;
        const addr_a& la;
        const addr_b& lb;
        unsigned int  rd; // LDS byte address of the stage the fragments are read from
        unsigned int  fill; // LDS byte address of this wave's block 0 in the stage the loads go to
        u32x4         rsrc_a, rsrc_b; // descriptors of the tile the loads fetch
    };

    // Which loads of a tile a step issues: loads BEGIN .. BEGIN+COUNT-1 (A's loads come
    // first, then B's), load BEGIN+v after MFMA FIRST + v * GAP.  The texture addresser
    // of the CU takes about 16 cycles per 1 KiB load; four waves that issue a load every
    // few MFMAs fill its queue and then stall in front of it, MFMAs included, so the
    // loads are spread as evenly as the ring allows.
    template<int FIRST, int GAP, int BEGIN, int COUNT>
    struct load_plan
    {
        static_assert(COUNT == 0 || FIRST + (COUNT - 1) * GAP < MFMAS, "loads must fit under the MFMAs of a step");
        static constexpr int first = FIRST, gap = GAP, begin = BEGIN, count = COUNT;
    };
    using no_loads = load_plan<0, 1, 0, 0>;

    // Scalar work of the caller's that wants a place among the MFMAs of a step: called
    // behind every MFMA with its number as a type.
    struct no_hook
    {
        template<class M>
        __device__ __forceinline__ void operator()(M) const
        {
        }
    };

    // MFMA number M of a step and the memory instructions that follow it: fragment
    // M / FRAG_GAP (A fragments first, then B) of K step READ_KK of the tile at c.rd
    // into (na, nb), and the load PLAN puts here, bound for c.fill.
    template<int M, int READ_KK, class PLAN, class HOOK>
    __device__ __forceinline__ static void slot(const step_ctx& c,
                                                const u32x4 (&fa)[TM],
                                                const u32x4 (&fb)[TN],
                                                u32x4 (&na)[TM],
                                                u32x4 (&nb)[TN],
                                                f32x4 (&acc)[TM][TN],
                                                const HOOK& hook)
    {
        constexpr bool HAS_LOAD = PLAN::count > 0 && M >= PLAN::first
                                  && (M - PLAN::first) % PLAN::gap == 0
                                  && (M - PLAN::first) / PLAN::gap < PLAN::count;
        if constexpr(HAS_LOAD)
        {
            constexpr int V = PLAN::begin + (M - PLAN::first) / PLAN::gap; // load of the tile
            if constexpr(V < op_a::PER_WAVE)
            {
                mfma_and_load<V * WAVES * 1024, (ONCE & 2) != 0>(acc[M / TN][M % TN], fa[M / TN], fb[M % TN], c.fill,
                                                c.la.template vector_offset<V>(), c.rsrc_a,
                                                V * c.la.stride);
            }
            else
            {
                constexpr int W = V - op_a::PER_WAVE;
                mfma_and_load<A_BYTES + W * WAVES * 1024, (ONCE & 1) != 0>(acc[M / TN][M % TN], fa[M / TN], fb[M % TN],
                                                          c.fill, c.lb.template vector_offset<W>(),
                                                          c.rsrc_b, W * c.lb.stride);
            }
        }
        else
        {
#ifdef RWG_SOLO_PROBE_HALF_MFMAS
            // Timing probe, results WRONG (never defined in a build that ships): the MFMAs
            // of the lower half of the wave tile that carry no load are left out, to see what
            // a pass over half a tile would cost with the loads and fragment reads unchanged.
            if constexpr(M / TN < TM / 2)
#endif
            mfma_16x16x32_pinned<IN>(acc[M / TN][M % TN], fa[M / TN], fb[M % TN]);
        }
        if constexpr(M % FRAG_GAP == 0 && M / FRAG_GAP < FRAGS)
        {
            constexpr int U = M / FRAG_GAP;
            if constexpr(U < TM)
            {
                na[U] = c.oa.template fragment_pinned<U, READ_KK>(c.rd);
            }
            else
            {
                nb[U - TM] = c.ob.template fragment_pinned<U - TM, READ_KK>(c.rd + A_BYTES);
            }
        }
        hook(std::integral_constant<int, M>{});
    }

    template<int READ_KK, class PLAN, class HOOK, int... M>
    __device__ __forceinline__ static void slots(std::integer_sequence<int, M...>,
                                                 const step_ctx& c,
                                                 const u32x4 (&fa)[TM],
                                                 const u32x4 (&fb)[TN],
                                                 u32x4 (&na)[TM],
                                                 u32x4 (&nb)[TN],
                                                 f32x4 (&acc)[TM][TN],
                                                 const HOOK& hook)
    {
        (slot<M, READ_KK, PLAN>(c, fa, fb, na, nb, acc, hook), ...);
    }

    // One K step: the MFMAs on (fa, fb) with the reads and loads between them.
    template<int READ_KK, class PLAN, class HOOK = no_hook>
    __device__ __forceinline__ static void step(const step_ctx& c,
                                                const u32x4 (&fa)[TM],
                                                const u32x4 (&fb)[TN],
                                                u32x4 (&na)[TM],
                                                u32x4 (&nb)[TN],
                                                f32x4 (&acc)[TM][TN],
                                                const HOOK& hook = HOOK{})
    {
        __builtin_amdgcn_sched_barrier(0);
        slots<READ_KK, PLAN>(
            std::make_integer_sequence<int, MFMAS>{}, c, fa, fb, na, nb, acc, hook);
        __builtin_amdgcn_sched_barrier(0);
    }

    // Loads V... of a tile without MFMAs around them (prologue).
    template<int... V>
    __device__ __forceinline__ static void issue_loads(std::integer_sequence<int, V...>,
                                                       const addr_a& la,
                                                       const addr_b& lb,
                                                       unsigned int  fill,
                                                       const u32x4&  rsrc_a,
                                                       const u32x4&  rsrc_b)
    {
        (
            [&] {
                if constexpr(V < op_a::PER_WAVE)
                {
                    load_only<V * WAVES * 1024>(fill, la.template vector_offset<V>(), rsrc_a, V * la.stride);
                }
                else
                {
                    constexpr int W = V - op_a::PER_WAVE;
                    load_only<A_BYTES + W * WAVES * 1024>(fill, lb.template vector_offset<W>(), rsrc_b,
                                                          W * lb.stride);
                }
            }(),
            ...);
    }

    // All fragments of K step 0 of the tile at LDS byte address rd.
    template<int... I, int... J>
    __device__ __forceinline__ static void read_first(std::integer_sequence<int, I...>,
                                                      std::integer_sequence<int, J...>,
                                                      const op_a&  oa,
                                                      const op_b&  ob,
                                                      unsigned int rd,
                                                      u32x4 (&fa)[TM],
                                                      u32x4 (&fb)[TN])
    {
        ((fa[I] = oa.template fragment_pinned<I, 0>(rd)), ...);
        ((fb[J] = ob.template fragment_pinned<J, 0>(rd + A_BYTES)), ...);
    }

    // Whole tiles: the wave's rows go through a private LDS strip so that a store
    // instruction writes 4 rows x 256 contiguous bytes (16 bytes per lane; 128-column wave tile) instead of
    // 16 rows x 32 bytes (16-bit C) or 16 rows x 64 bytes (fp32 C and partial sums; the
    // strip is worth 6..9 % at 8192^3 and 13..16 % with shorter K there).  At 4096^3 the
    // C stores are 11 % of the call.  STREAM marks the stores as streaming: C is not read
    // again here, and without the hint the 4 MiB of C that the workgroups of an XCD write
    // at the same time push the operand panels out of its L2 (+3..5 % with several tiles
    // per workgroup, nothing lost with one).  Strip: 16 rows
    // at a pitch of 272 bytes (the 8-byte writes of a half-wave then fall on 32 distinct
    // 8-byte bank columns; the 16-byte reads take two cycles instead of one, which does
    // not show).  LDS operations of one wave are served in order, so the reads see the
    // writes without a barrier; the waits keep the compiler from reordering them.
    static constexpr int ROW_BYTES   = TN * 32; // 256 for the 128-column wave tile
    static constexpr int STRIP_PITCH = ROW_BYTES + 16;
    static constexpr int STRIP_BYTES = (16 * STRIP_PITCH + 1023) / 1024 * 1024;
    static_assert(LDS_BYTES + WAVES * STRIP_BYTES + WAVES * 256 <= 160 * 1024,
                  "tile ring, store strips and the sink of the line touches must fit the 160 KB LDS");

    // Ties a row of accumulators to its registers at this point of the program: what
    // follows reads the row from there.  Without it the compiler copies all 256
    // accumulator registers into ordinary ones right behind the K loop, where there is
    // no room for them, and spills.
    __device__ __forceinline__ static void pin_row(f32x4 (&row)[TN])
    {
        static_assert(TN % 2 == 0, "two accumulators per statement");
#pragma unroll
        for(int j = 0; j < TN; j += 2)
        {
            asm volatile("" : "+a"(row[j]), "+a"(row[j + 1]));
        }
    }

    // The stores are buffer stores relative to the tile's origin: the part of the address
    // that is the same for the whole wave goes into the scalar offset, the lane's part is
    // computed once per call, and a lane whose piece lies in a row >= rows or a column >=
    // cols of the tile (GUARDED: a tile on a ragged edge) gets an offset beyond the
    // descriptor's 2 GiB range, so the hardware drops its store: no branch, the same code
    // for every tile.  cols is a multiple of a piece's width (the host sends a C whose
    // rows are not 16-byte aligned, or whose width is no multiple of 8, to another
    // kernel), so a piece lies inside or outside as a whole; a tile's rows span less than
    // 2 GiB (the host checks), so scalar + vector offset neither wraps nor, for a dropped
    // lane, comes back into range.
    static constexpr unsigned int STORE_RANGE = 0x80000000u;

    // (the compiler's own buffer store: it knows how long the store reads its data
    // registers and keeps the next write to them away)
    template<bool STREAM>
    __device__ __forceinline__ static void store_piece(const u32x4& v, unsigned int lane_offset,
                                                       __amdgpu_buffer_rsrc_t rsrc, unsigned int wave_offset)
    {
        __builtin_amdgcn_raw_buffer_store_b128(v, rsrc, lane_offset, wave_offset, STREAM ? 2 : 0); // 2 = nt
    }

    template<bool STREAM, bool GUARDED, class DstT>
    __device__ __forceinline__ static void write_out_staged(f32x4 (&acc)[TM][TN],
                                                            DstT*        tile, // element (0, 0) of the workgroup's tile
                                                            long long    pitch,
                                                            int          rows, // of the tile that exist
                                                            int          cols,
                                                            int          row_w, // the wave's corner in the tile
                                                            int          col_w,
                                                            int          lane,
                                                            lds_char_ptr strip)
    {
        // a strip row holds ROW_BYTES: all columns of the wave tile for a 16-bit
        // destination, half of them for fp32
        constexpr int PASSES = sizeof(DstT) / 2;
        static_assert(TN % PASSES == 0, "whole tiles per pass");
        constexpr int TILES   = TN / PASSES; // 16-column tiles per pass
        constexpr int CHUNKS  = ROW_BYTES / 16; // 16-byte pieces of a strip row
        constexpr int READS   = 16 * CHUNKS / 64; // store instructions per pass
        constexpr int PIECE   = 16 / (int)sizeof(DstT); // elements of a piece
        static_assert(16 * CHUNKS % 64 == 0, "the strip divides over the lanes");
        typedef DstT out4 __attribute__((ext_vector_type(4)));
        using lds_out4  = __attribute__((address_space(3))) out4;
        using lds_u32x4 = __attribute__((address_space(3))) u32x4;
        // (the tile's origin is the same in every lane; see scalar_pointer)
        const unsigned long long base = (unsigned long long)tile;
        // (readfirstlane returns a signed int: through unsigned int, or the low half's
        // sign bit smears over the high half)
        const unsigned int lo = (unsigned int)__builtin_amdgcn_readfirstlane((unsigned int)base);
        const unsigned int hi = (unsigned int)__builtin_amdgcn_readfirstlane((unsigned int)(base >> 32));
        const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
            (void*)(((unsigned long long)hi << 32) | (unsigned long long)lo), 0, (int)STORE_RANGE, 0x00020000);
        const int                r16 = lane & 15, g = lane >> 4;
        // this lane's piece of read q: row and column in the 16-row block, strip address,
        // offset in the destination
        int          piece_row[READS], piece_col[READS], strip_at[READS];
        unsigned int piece_off[READS];
#pragma unroll
        for(int q = 0; q < READS; ++q)
        {
            const int piece = q * 64 + lane;
            piece_row[q]    = piece / CHUNKS;
            piece_col[q]    = piece % CHUNKS * PIECE;
            strip_at[q]     = piece_row[q] * STRIP_PITCH + piece % CHUNKS * 16;
            piece_off[q]    = (unsigned int)((piece_row[q] * pitch + piece_col[q]) * (long long)sizeof(DstT));
        }
#pragma unroll
        for(int i = 0; i < TM; ++i)
        {
            pin_row(acc[i]);
#pragma unroll
            for(int p = 0; p < PASSES; ++p)
            {
#pragma unroll
                for(int j = 0; j < TILES; ++j)
                {
                    out4 o;
#pragma unroll
                    for(int v = 0; v < 4; ++v)
                    {
                        o[v] = to_out<DstT>(acc[i][p * TILES + j][v]);
                    }
                    *reinterpret_cast<lds_out4*>(strip + r16 * STRIP_PITCH + (16 * j + 4 * g) * sizeof(DstT)) = o;
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                const int          row0 = row_w + 16 * i, col0 = col_w + p * TILES * 16; // of the block
                const unsigned int wave_offset = __builtin_amdgcn_readfirstlane(
                    (unsigned int)((row0 * pitch + col0) * (long long)sizeof(DstT)));
#pragma unroll
                for(int q = 0; q < READS; ++q)
                {
                    const u32x4  v      = *reinterpret_cast<lds_u32x4*>(strip + strip_at[q]);
                    unsigned int offset = piece_off[q];
                    if constexpr(GUARDED)
                    {
                        offset = row0 + piece_row[q] < rows && col0 + piece_col[q] < cols ? offset : STORE_RANGE;
                    }
                    store_piece<STREAM>(v, offset, rsrc, wave_offset);
                }
                asm volatile("" ::: "memory");
            }
        }
    }

    // One unit of work of a workgroup: a C tile, or a run of K tiles of one, of one batch
    // entry.
    struct work_item
    {
        int        batch;
        int        row0, col0;
        int        nk; // K tiles, at least one
        int        cls; // tile row + tile column: which K tile of a group the item starts at (args.k_group)
        const InT* a; // first K tile of the operands
        const InT* b;
        const InT* a_end; // where the loads' range ends (see limits)
        const InT* b_end;
        bool       ends_k; // the item's last K tile is the last of K
        float*     partial; // nullptr: the item is a whole tile and goes to C; else where
                            // element (row, col) of C, global coordinates, goes:
                            // partial[row * pitch + col]
        long long  pitch;
        int        next; // position of the workgroup's next item
    };

    // The items of a workgroup, in one of two orders.
    //  - by item (args.stream_units == 0): the launch holds blocks_per_batch * batches
    //    items (whole tiles first, then K slices of the split tiles, per batch entry);
    //    a position is an item number and workgroup g takes g, g + gridDim.x, ...
    //  - by K tile (args.stream_units = U > 0): all K tiles of all tiles of all batch
    //    entries form one sequence, tile after tile in walk order, and workgroup g takes
    //    K tiles [g * U, (g + 1) * U) of it: every workgroup does the same number of
    //    MFMAs whatever the tile count.  A position is a K tile number; an item is the
    //    part of the workgroup's range that lies in one tile.  A tile that lies in one
    //    range goes to C; of a tile cut by range borders every part goes to the
    //    workgroup's first or second fp32 slot ("first": the part holds the range's first
    //    K tile) and reduce_stream_tiles adds the parts up.
    struct walk
    {
        int begin, end, hop; // positions of this workgroup: begin, then item.next, while < end

        __device__ __forceinline__ static walk of(const gemm_args& args)
        {
            if(args.stream_units == 0)
            {
                return {(int)blockIdx.x, args.blocks_per_batch * args.batches, (int)gridDim.x};
            }
            const int total = args.grid_m * args.grid_n * args.batches * (args.K / BK);
            const int begin = blockIdx.x * args.stream_units;
            const int end   = begin + args.stream_units;
            return {begin, end < total ? end : total, 0};
        }
    };

    __device__ __forceinline__ static work_item decode(const gemm_args& args, const walk& wk, int pos)
    {
        work_item x;
        const int k_steps_total = args.K / BK;
        int       step_begin;
        if(wk.hop != 0)
        {
            // (positions that are congruent mod 8 run on the same XCD: the grid is a
            // multiple of 8 workgroups whenever a workgroup takes more than one position)
            const int item     = args.batch_by_xcd ? xcd_remap(pos, wk.end) : pos;
            x.batch            = item / args.blocks_per_batch;
            const block_work w = decode_block(args, item - x.batch * args.blocks_per_batch);
            const tile_coord t = args.batch_by_xcd
                                     ? banded_tile(w.tile_id, args.grid_m, args.grid_n, args.group)
                                     : map_tile(w.tile_id, args.grid_m, args.grid_n, args.group);
            x.row0             = t.m * BM;
            x.col0             = t.n * BN;
            const int steps_per = (k_steps_total + w.slices - 1) / w.slices;
            step_begin          = w.slice * steps_per;
            int step_end        = step_begin + steps_per;
            if(step_end > k_steps_total)
            {
                step_end = k_steps_total;
            }
            x.nk      = step_end - step_begin;
            x.next    = pos + wk.hop;
            x.partial = nullptr;
            x.pitch   = args.N;
            if(w.slices > 1)
            {
                x.partial = partial_base<BM, BN>(args, w, x.batch, x.row0, x.col0, x.pitch);
            }
        }
        else
        {
            const int tiles    = args.grid_m * args.grid_n;
            const int tile_lin = pos / k_steps_total;
            step_begin         = pos - tile_lin * k_steps_total;
            x.batch            = tile_lin / tiles;
            const tile_coord t = map_tile(tile_lin - x.batch * tiles, args.grid_m, args.grid_n, args.group);
            x.row0             = t.m * BM;
            x.col0             = t.n * BN;
            x.nk               = k_steps_total - step_begin;
            if(x.nk > wk.end - pos)
            {
                x.nk = wk.end - pos;
            }
            x.next    = pos + x.nk;
            x.partial = nullptr;
            x.pitch   = args.N;
            if(x.nk != k_steps_total)
            {
                const long long slot = 2 * (long long)blockIdx.x + (pos == wk.begin ? 0 : 1);
                x.partial = args.partials + slot * (long long)(BM * BN) - ((long long)x.row0 * BN + x.col0);
                x.pitch   = BN;
            }
        }
        const long long a_sr = A_KMAJOR ? args.lda : 1, a_sk = A_KMAJOR ? 1 : args.lda;
        const long long b_sr = B_KMAJOR ? args.ldb : 1, b_sk = B_KMAJOR ? 1 : args.ldb;
        // The integer divisions above run on the vector ALU (there is no scalar divide),
        // and the compiler then tends to keep what depends on them in vector registers;
        // the buffer descriptors built from these pointers must be scalar.
        x.a = scalar_pointer(static_cast<const InT*>(args.A) + x.batch * args.batch_stride_a
                             + x.row0 * a_sr + (long long)step_begin * BK * a_sk);
        x.b = scalar_pointer(static_cast<const InT*>(args.B) + x.batch * args.batch_stride_b
                             + x.col0 * b_sr + (long long)step_begin * BK * b_sk);
        x.ends_k = step_begin + x.nk == k_steps_total;
        x.cls    = __builtin_amdgcn_readfirstlane(x.row0 / BM + x.col0 / BN);
        limits(args, x);
        return x;
    }

    // Where the range of an item's load descriptors ends (guarded kernels only; the
    // others do not check).  A K-contiguous operand: at the end of the allocation (the
    // last batch entry's last row).  An M/N-contiguous operand: at the end of the item's
    // batch entry, which is the end of its K rows, so that the rows of the last K tile
    // past K read zeros in every batch entry.
    __device__ __forceinline__ static void limits(const gemm_args& args, work_item& x)
    {
        if constexpr(GUARD_C)
        {
            const long long k_rows = args.K - (args.k_tail ? BK - args.k_tail : 0);
            x.a_end = scalar_pointer(static_cast<const InT*>(args.A)
                                     + (A_KMAJOR ? (args.batches - 1) * args.batch_stride_a + args.M * args.lda
                                                 : x.batch * args.batch_stride_a + k_rows * args.lda));
            x.b_end = scalar_pointer(static_cast<const InT*>(args.B)
                                     + (B_KMAJOR ? (args.batches - 1) * args.batch_stride_b + args.N * args.ldb
                                                 : x.batch * args.batch_stride_b + k_rows * args.ldb));
        }
        else
        {
            x.a_end = nullptr;
            x.b_end = nullptr;
        }
    }

    // The accumulators of a finished work item, to C or to the fp32 partial tiles.
    __device__ __forceinline__ static void write_item(const gemm_args&   args,
                                                      const work_item&   x,
                                                      f32x4 (&acc)[TM][TN],
                                                      int                row_w,
                                                      int                col_w,
                                                      int                lane,
                                                      lds_char_ptr       strip)
    {
        if(x.partial == nullptr)
        {
            OutT* C = static_cast<OutT*>(args.C) + x.batch * args.batch_stride_c + (long long)x.row0 * args.N + x.col0;
            write_out_staged<true, GUARD_C>(acc, C, args.N, args.M - x.row0, args.N - x.col0, row_w, col_w, lane,
                                            strip);
        }
        else
        {
            // The reduce kernel reads these next: no streaming hint.  A tile of its own
            // has nothing to leave out; whole planes of a ragged C do.
            const bool own_tile = args.tail_begin != 0 || args.stream_units != 0;
            write_out_staged<false, GUARD_C>(acc, x.partial + (long long)x.row0 * x.pitch + x.col0, x.pitch,
                                             own_tile ? BM : args.M - x.row0, own_tile ? BN : args.N - x.col0,
                                             row_w, col_w, lane, strip);
        }
    }

    // Makes the zeroed accumulators safe to feed to the hand-written MFMAs: the compiler
    // does not see that those read them, so it would not keep the wait states between
    // the writes and the first read.
    __device__ __forceinline__ static void settle_row(f32x4 (&row)[TN])
    {
        static_assert(TN % 2 == 0, "two accumulators per statement");
#pragma unroll
        for(int j = 0; j < TN; j += 2)
        {
            asm volatile("s_nop 4" : "+a"(row[j]), "+a"(row[j + 1]));
        }
    }

    // The workgroups are persistent: a workgroup works on its items (see walk) one after
    // the other, and the K tiles of all its items form ONE stream through the ring, so
    // the loads of an item's first two K tiles go out under the last two steps of the
    // item before it and the only thing between two items' MFMAs is the store of the
    // accumulators.  (A workgroup per item pays, per item, the dispatch of the next
    // workgroup, the latency of the first loads and the drain of the stores: about
    // 13 us, nine K tiles' worth, at 256 x 256 x 64.)
    __device__ __forceinline__ static void run(const gemm_args& args)
    {
        __shared__ __attribute__((aligned(1024))) char lds_raw[LDS_BYTES + WAVES * STRIP_BYTES + WAVES * 256];
        lds_char_ptr lds = (lds_char_ptr)lds_raw;

        const int tid    = threadIdx.x;
        const int lane   = tid & 63;
        const int wave   = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int wave_m = wave / WAVES_N;
        const int wave_n = wave % WAVES_N;

        const walk wk = walk::of(args);

        const long long a_ld   = args.lda;
        const long long b_ld   = args.ldb;
        const long long a_step = BK * (A_KMAJOR ? 1 : a_ld), b_step = BK * (B_KMAJOR ? 1 : b_ld);

        op_a oa;
        op_b ob;
        oa.init(wave, lane, a_ld, wave_m * WTM);
        ob.init(wave, lane, b_ld, wave_n * WTN);
        addr_a la;
        addr_b lb;
        la.init(wave, lane, a_ld);
        lb.init(wave, lane, b_ld);

        // a last K tile that the operands hold only in part (guarded kernels)
        const bool   k_ragged = GUARD_C && args.k_tail != 0;
        const addr_a la_tail  = la.for_tail(lane, wave, args.k_tail);
        const addr_b lb_tail  = lb.for_tail(lane, wave, args.k_tail);

        work_item cur = decode(args, wk, wk.begin);

        // The stream of K tiles the loads follow; it runs two tiles ahead of the MFMAs.
        // Past the last item it wraps to the workgroup's first item, so the last two
        // tiles' worth of loads fetch that item's K tiles 0 and 1 again into stages nobody
        // reads.  That keeps the loop uniform, and it is kept on purpose: switching those
        // loads off (tried with a branch per load and with a zero-sized buffer descriptor)
        // made back-to-back calls on the same operands 5 % slower at 4096^3, because the
        // 32 workgroups of an XCD leave exactly the first two K tiles of their operand
        // panels in its 4 MiB L2 for the next call; a call on fresh operands pays two
        // tiles of extra L2 -> LDS traffic for nothing.
        const InT* a_src       = cur.a;
        const InT* b_src       = cur.b;
        const InT* a_end       = cur.a_end;
        const InT* b_end       = cur.b_end;
        int        stream_left = cur.nk;
        int        stream_next = cur.next;
        bool       stream_ends = cur.ends_k;
        // The order of an item's K tiles in the kernels built with K_RUNS (args.k_block = b, a
        // power of two): runs of b tiles; within every 8 runs the workgroups of XCD x take
        // run x first, then x + 1, ... and wrap round.
        // Workgroups that all walk K in step make every XCD that needs a panel ask for the
        // same lines at the same moment, so every L2 miss waits for HBM (a fabric read took
        // 850 cycles against 620 for a kernel whose XCDs are not in step, and with operands
        // beyond the 256 MB memory-side cache that wait is what bounds the K loop: each CU
        // has only so many lines in flight).  Out of step by whole runs, each XCD is the first
        // to ask memory for a share of the runs of a panel and finds the others in the
        // memory-side cache, fetched by the XCD that was there first; and unlike a constant
        // offset between XCDs, which leaves one XCD first everywhere and as slow as before,
        // the roles change with every run.  The workgroups of ONE XCD still walk in step:
        // they share panels through its L2.  4096 x 4096 x 28672 bf16 with both operands
        // K-contiguous 1235 -> 1365 TFLOP/s, 8192 x 8192 x 28672 1250 -> 1340; nothing
        // gained where the operands fit that cache, and the bookkeeping costs 1..2 % there,
        // hence a kernel of its own.  An operand that is contiguous along M or N never had
        // the problem (a k row of a tile is four whole lines).
        // The same one level down (args.k_group = g): within every aligned group of g K tiles
        // the workgroup of tile (i, j) starts at tile (i + j) mod g and wraps round.  The 8
        // workgroups of an XCD that share an A panel (a tile row) and the 4 that share a B
        // panel (a tile column) then ask for a line at g different times: the first waits for
        // the fabric, the others find the line in L2 instead of queueing behind the same
        // miss, and a compute unit's lines in flight turn over that much faster (the XCD's
        // L2 holds the g K tiles of its 12 panels: 1.5 MB of 4 at g = 4).  By tile row or by
        // tile column alone it is worth half as much, and a constant offset (every row a K
        // tile further on, all the way) nothing: whoever is ahead stays ahead and as slow
        // as before.  4096 x 4096 x 28672 bf16, both operands K-contiguous: 1240 -> 1440
        // TFLOP/s with g = 4, 1480 with g = 8 (1365 with the runs by XCD alone, 1425 with
        // runs and groups; the vendor kernel of the same tile 1525), 8192 x 8192 x 28672
        // 1250 -> 1460 (1530).  Where the operands fit the memory-side cache the plain walk is
        // level or ahead (8192^3 1590 against 1580, 4096^3 1490 against 1460).
        // (Written without branches, masks that are zero where an order does not apply, so that
        // the few scalar instructions sit among the MFMAs instead of in blocks of their own.)
        const int  perm_xcd    = (int)(blockIdx.x & 7);
        const int  perm_span   = K_RUNS ? 8 * args.k_block : 0; // K tiles of 8 runs (0: in order)
        const int  perm_shift  = K_RUNS && args.k_block > 0 ? 31 - __builtin_clz((unsigned int)args.k_block) : 0;
        const int  span_mask   = perm_span > 0 ? perm_span - 1 : 0;
        const int  run_mask    = K_RUNS && args.k_block > 0 ? args.k_block - 1 : 0;
        const int  group_mask  = K_RUNS && args.k_group > 0 ? args.k_group - 1 : 0;
        int        stream_t    = 0; // place in the walk
        int        stream_k    = 0; // K tile there
        int        stream_nk   = cur.nk;
        const InT* a_item      = cur.a;
        const InT* b_item      = cur.b;
        int        stream_cls  = cur.cls;
        const int  runs_apply  = perm_span != 0 ? ~span_mask : 0;
        // (the last tiles that do not fill a group are walked as they are)
        auto in_group = [&](int t, int nk, int cls) {
            const int gm = t < (nk & ~group_mask) ? group_mask : 0;
            return (t & ~gm) | ((t + cls) & gm);
        };
        // (the last runs that do not fill a group of 8 are walked as they are; none at all when
        // there are no runs)
        auto in_runs = [&](int k, int nk) {
            const int r  = k & span_mask;
            const int kr = (k - r) + (((((r >> perm_shift) + perm_xcd) & 7) << perm_shift) | (r & run_mask));
            return k < (nk & runs_apply) ? kr : k;
        };
        auto k_of = [&](int t, int nk, int cls) { return in_runs(in_group(t, nk, cls), nk); };
        if constexpr(K_RUNS)
        {
            stream_k = k_of(0, stream_nk, stream_cls);
            a_src += stream_k * a_step;
            b_src += stream_k * b_step;
        }
        // Line touches (args.warm_ahead = distance in K tiles, + 4 for "every workgroup touches
        // whole tiles"): which quarter of a K tile's lines this workgroup touches.  The
        // workgroups that share an A panel differ in their tile column, those that share a B
        // panel in their tile row, so a run of four neighbours covers a tile; wave 0 touches
        // A's lines, wave 1 B's.  With whole tiles, wave w touches quarter w of both.
        const int          warm_dist = args.warm_ahead & 3;
        const bool         warm_full = (args.warm_ahead & 4) != 0;
        const unsigned int lds_sink  = (unsigned int)(size_t)lds + LDS_BYTES + WAVES * STRIP_BYTES + wave * 256;
        // K-contiguous: lane l touches the line of row 4 l + quarter (a row of a K tile is one
        // line); else lane l touches line `quarter` of k row l (four lines of 128 bytes hold
        // the 256 elements of a k row)
        const unsigned int warm_voff_a = (unsigned int)((A_KMAJOR ? 4 * lane : lane) * a_ld * 2);
        const unsigned int warm_voff_b = (unsigned int)((B_KMAJOR ? 4 * lane : lane) * b_ld * 2);
        const InT* warm_end_a = scalar_pointer(static_cast<const InT*>(args.A) + (args.batches - 1) * args.batch_stride_a
                                               + (A_KMAJOR ? (long long)args.M * a_ld : (long long)args.K * a_ld));
        const InT* warm_end_b = scalar_pointer(static_cast<const InT*>(args.B) + (args.batches - 1) * args.batch_stride_b
                                               + (B_KMAJOR ? (long long)args.N * b_ld : (long long)args.K * b_ld));
        // (scalar by hand: the tile coordinates come out of vector divisions)
        auto quarters_of = [&](const work_item& x) {
            const unsigned int qa = warm_full ? wave : (x.col0 / BN) & 3, qb = warm_full ? wave : (x.row0 / BM) & 3;
            return (unsigned int)__builtin_amdgcn_readfirstlane(qa | (qb << 8));
        };
        unsigned int stream_quarters = quarters_of(cur);
        // Where the order puts the tile after the current one, worked out ahead of advance():
        // in the K loop from among the MFMAs of the second step (the scalar instructions cost
        // nothing there; behind the last MFMA they are 3..4 % of a tile's time).
        int        k_next = 0;
        const InT* a_next = a_src;
        const InT* b_next = b_src;
        auto plan_next = [&](auto part) {
            if constexpr(K_RUNS)
            {
                constexpr int PART = decltype(part)::value; // (-1: all of it)
                if constexpr(PART == 0 || PART == -1)
                {
                    k_next = in_group(stream_t + 1, stream_nk, stream_cls);
                }
                if constexpr(PART == 1 || PART == -1)
                {
                    k_next = in_runs(k_next, stream_nk);
                }
                if constexpr(PART == 2 || PART == -1)
                {
                    a_next = a_item + k_next * a_step;
                }
                if constexpr(PART == 3 || PART == -1)
                {
                    b_next = b_item + k_next * b_step;
                }
            }
        };
        constexpr std::integral_constant<int, -1> whole{};
        auto advance = [&]() {
            if constexpr(K_RUNS)
            {
                ++stream_t;
                stream_k = k_next;
                a_src    = a_next;
                b_src    = b_next;
            }
            else
            {
                a_src += a_step;
                b_src += b_step;
            }
            if(--stream_left == 0)
            {
                const work_item nx = decode(args, wk, stream_next < wk.end ? stream_next : wk.begin);
                a_src              = nx.a;
                b_src              = nx.b;
                a_end              = nx.a_end;
                b_end              = nx.b_end;
                stream_left        = nx.nk;
                stream_next        = nx.next;
                stream_ends        = nx.ends_k;
                stream_quarters    = quarters_of(nx);
                if constexpr(K_RUNS)
                {
                    a_item     = nx.a;
                    b_item     = nx.b;
                    stream_nk  = nx.nk;
                    stream_t   = 0;
                    stream_cls = nx.cls;
                    stream_k   = k_of(0, nx.nk, nx.cls);
                    a_src      = nx.a + stream_k * a_step;
                    b_src      = nx.b + stream_k * b_step;
                }
            }
        };
        // whether the tile at (a_src, b_src) is a last K tile held only in part (the item's
        // last tile in K order, wherever the walk has it)
        auto partial_tile = [&]() {
            return k_ragged && stream_ends && (K_RUNS ? stream_k == stream_nk - 1 : stream_left == 1);
        };

        const unsigned int lds_addr   = (unsigned int)(size_t)lds;
        const unsigned int wave_block = lds_addr + wave * 1024; // this wave's block 0, stage 0
        lds_char_ptr       strip      = lds + LDS_BYTES + wave * STRIP_BYTES;
        u32x4 fa[2][TM], fb[2][TN];

        if constexpr(STAGES == 4)
        {
            // Ring of 4 tiles of one K step each.  The fragments of tile t+1 are read under
            // the MFMAs of tile t, so tile t's stage is free when all waves have arrived at
            // the barrier in front of tile t, and the loads of tile t+4 go out under tile t:
            // a load has between two and three tiles' time to land (one quarter to one with
            // the ring of 2), at the price of a barrier per K step instead of one per two.
            using plan = load_plan<2, (MFMAS - 2) / VM_LOADS, 0, VM_LOADS>;
            constexpr unsigned int RING = STAGES * STAGE;
#pragma unroll
            for(int s = 0; s < STAGES; ++s)
            {
                const bool part = partial_tile();
                issue_loads(std::make_integer_sequence<int, VM_LOADS>{}, la.or_else(part, la_tail),
                            lb.or_else(part, lb_tail), wave_block + s * STAGE, descriptor(a_src, a_end),
                            descriptor(b_src, b_end));
                plan_next(whole);
                advance();
            }
            __builtin_amdgcn_s_waitcnt(waitcnt_imm(3 * VM_LOADS));
            __builtin_amdgcn_s_barrier();
            read_first(std::make_integer_sequence<int, TM>{}, std::make_integer_sequence<int, TN>{},
                       oa, ob, lds_addr, fa[0], fb[0]);

            unsigned int here = 0; // stage (byte offset) of the tile the MFMAs are on
            // One tile: wait for the own loads of the next tile (the loads of the two tiles
            // behind it stay in flight) and the own fragment reads of this one, barrier, then
            // the MFMAs with the next tile's fragment reads and the loads of the tile four on.
            auto tile_step = [&](const u32x4 (&ca)[TM], const u32x4 (&cb)[TN], u32x4 (&na)[TM], u32x4 (&nb)[TN],
                                 f32x4 (&acc)[TM][TN]) {
                const unsigned int there = here + STAGE == RING ? 0 : here + STAGE;
                const bool         part  = partial_tile();
                const addr_a       la1   = la.or_else(part, la_tail);
                const addr_b       lb1   = lb.or_else(part, lb_tail);
                const step_ctx     c{oa, ob, la1, lb1, lds_addr + there, wave_block + here,
                                     descriptor(a_src, a_end), descriptor(b_src, b_end)};
                __builtin_amdgcn_s_waitcnt(waitcnt_imm(2 * VM_LOADS));
                __builtin_amdgcn_s_barrier();
                step<0, plan>(c, ca, cb, na, nb, acc);
                plan_next(whole);
                advance();
                here = there;
            };
            for(;;)
            {
                f32x4 acc[TM][TN];
#pragma unroll
                for(int i = 0; i < TM; ++i)
                {
#pragma unroll
                    for(int j = 0; j < TN; ++j)
                    {
                        acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                    }
                }
#pragma unroll
                for(int i = 0; i < TM; ++i)
                {
                    settle_row(acc[i]);
                }
                for(int it = 0;;)
                {
                    tile_step(fa[0], fb[0], fa[1], fb[1], acc);
                    if(++it == cur.nk)
                    {
                        break;
                    }
                    tile_step(fa[1], fb[1], fa[0], fb[0], acc);
                    if(++it == cur.nk)
                    {
                        break;
                    }
                }
                // (the fragments read under the last step belong to the next item; they are
                // read again behind the stores, which need the registers)
                asm volatile("s_waitcnt lgkmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");
                write_item(args, cur, acc, wave_m * WTM, wave_n * WTN, lane, strip);
                if(cur.next >= wk.end)
                {
                    break;
                }
                cur = decode(args, wk, cur.next);
                read_first(std::make_integer_sequence<int, TM>{}, std::make_integer_sequence<int, TN>{},
                           oa, ob, lds_addr + here, fa[0], fb[0]);
            }
        }
        else
        {
        // Ring of 2 tiles, two K steps per tile.  Tile t: first step on K step 0 with
        // the reads of K step 1; then wait for the own loads of tile t+1 and the own
        // reads of tile t, barrier; second step on K step 1 with the reads of tile
        // t+1's K step 0.  Tile t's stage is free from that barrier on: the loads of
        // tile t+2 go out under the second step (three quarters of them) and the
        // first quarter of tile t+1's first step.
        constexpr int LOADS_A = VM_LOADS * RWG_SOLO_LATE_LOADS_16THS / 16, LOADS_B = VM_LOADS - LOADS_A;
        using plan_b = load_plan<2, (MFMAS - 2) / LOADS_B, 0, LOADS_B>;
        using plan_a = load_plan<1, RWG_SOLO_LATE_GAP, LOADS_B, LOADS_A>;
        // prologue: tile 0 and the first part of tile 1 on their way, tile 0 landed
        {
            const bool part = partial_tile();
            issue_loads(std::make_integer_sequence<int, VM_LOADS>{}, la.or_else(part, la_tail),
                        lb.or_else(part, lb_tail), wave_block, descriptor(a_src, a_end), descriptor(b_src, b_end));
        }
        plan_next(whole);
        advance();
        bool part_prev = partial_tile();
        issue_loads(std::make_integer_sequence<int, LOADS_B>{}, la.or_else(part_prev, la_tail),
                    lb.or_else(part_prev, lb_tail), wave_block + STAGE, descriptor(a_src, a_end),
                    descriptor(b_src, b_end));
        const InT* a_prev     = a_src;
        const InT* b_prev     = b_src;
        const InT* a_end_prev = a_end;
        const InT* b_end_prev = b_end;
        plan_next(whole);
        advance();
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(LOADS_B));
        __builtin_amdgcn_s_barrier();
        read_first(std::make_integer_sequence<int, TM>{}, std::make_integer_sequence<int, TN>{},
                   oa, ob, lds_addr, fa[0], fb[0]);

        unsigned int here = 0; // stage (byte offset) of the tile the MFMAs are on
        for(;;)
        {
            f32x4 acc[TM][TN];
#pragma unroll
            for(int i = 0; i < TM; ++i)
            {
#pragma unroll
                for(int j = 0; j < TN; ++j)
                {
                    acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                }
            }
#pragma unroll
            for(int i = 0; i < TM; ++i)
            {
                settle_row(acc[i]);
            }

            for(int it = 0; it < cur.nk; ++it)
            {
                const unsigned int there = STAGE - here;
                const bool     part = partial_tile();
                const addr_a   la0 = la.or_else(part_prev, la_tail), la1 = la.or_else(part, la_tail);
                const addr_b   lb0 = lb.or_else(part_prev, lb_tail), lb1 = lb.or_else(part, lb_tail);
                const step_ctx c0{oa, ob, la0, lb0, lds_addr + here, wave_block + there,
                                  descriptor(a_prev, a_end_prev), descriptor(b_prev, b_end_prev)};
                const step_ctx c1{oa, ob, la1, lb1, lds_addr + there, wave_block + here,
                                  descriptor(a_src, a_end), descriptor(b_src, b_end)};
                __builtin_amdgcn_s_waitcnt(waitcnt_imm(63)); // last step's fragment reads
                step<1, plan_a>(c0, fa[0], fb[0], fa[1], fb[1], acc);
                __builtin_amdgcn_s_waitcnt(waitcnt_imm(0));
                __builtin_amdgcn_s_barrier();
                // (and of the same run, where the K tiles are walked in runs)
                if(warm_dist != 0 && stream_left > warm_dist
                   && (perm_span == 0 || (stream_t & (args.k_block - 1)) + warm_dist < args.k_block)
                   && args.k_group == 0)
                {
                    // a K tile further down the stream than the one whose loads follow, if it
                    // is the same item's
                    if(warm_full || wave == 0)
                    {
                        touch_lines(lds_sink, warm_voff_a, a_src + warm_dist * a_step, warm_end_a,
                                    (unsigned int)__builtin_amdgcn_readfirstlane((unsigned int)(
                                        (stream_quarters & 255) * (A_KMAJOR ? a_ld * 2 : 128))));
                    }
                    if(warm_full || wave == 1)
                    {
                        touch_lines(lds_sink, warm_voff_b, b_src + warm_dist * b_step, warm_end_b,
                                    (unsigned int)__builtin_amdgcn_readfirstlane((unsigned int)(
                                        (stream_quarters >> 8) * (B_KMAJOR ? b_ld * 2 : 128))));
                    }
                }
                step<0, plan_b>(c1, fa[1], fb[1], fa[0], fb[0], acc, [&](auto m) {
                    // (a few scalar instructions behind each of four MFMAs)
                    constexpr int AT = decltype(m)::value;
                    if constexpr(AT >= 4 && AT <= 16 && AT % 4 == 0)
                    {
                        plan_next(std::integral_constant<int, AT / 4 - 1>{});
                    }
                });
                a_prev     = a_src;
                b_prev     = b_src;
                a_end_prev = a_end;
                b_end_prev = b_end;
                part_prev  = part;
                advance();
                here = there;
            }
            // the MFMAs are invisible to the compiler, so cover their result latency by
            // hand; the next item's first fragments and loads stay in flight
            asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
            write_item(args, cur, acc, wave_m * WTM, wave_n * WTN, lane, strip);

            if(cur.next >= wk.end)
            {
                break;
            }
            cur = decode(args, wk, cur.next);
            // The last step read these fragments already; reading them again here instead
            // of keeping them across the stores leaves the stores the registers (with 64
            // more live the compiler spilled accumulators to scratch memory).
            read_first(std::make_integer_sequence<int, TM>{}, std::make_integer_sequence<int, TN>{},
                       oa, ob, lds_addr + here, fa[0], fb[0]);
        }
        }
        // the wrapped tail loads are still in flight
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(0));
    }
};

} // namespace device
} // namespace rocm_wmma_gemm

#endif // ROCM_WMMA_GEMM_SOLO_KERNEL_HPP
