// Whole-K streaming MFMA GEMM kernel for gfx950: small output tiles (16, 32 or 64 rows and
// columns), one workgroup per tile, the whole K range inside the workgroup, for problems
// that are bound by the stream of one operand from HBM (a skinny M or N against a large
// N x K or M x K operand: decode-like shapes).
//
// What it is for.  A 16 x 8192 x 8192 GEMM reads 134 MB of B and does almost no arithmetic.
// With 256 x 256 tiles it has 32 tiles for 256 compute units; the other kernels therefore
// cut K into slices, write fp32 partial planes and add them up in a second launch, which
// costs a quarter of the call.  Here the tiles are small enough that N / 32 of them cover
// every compute unit without cutting K, so one launch does the whole job and the sums
// keep one fixed order:
//   - a workgroup streams its 32 (or 64) rows of the large operand from HBM exactly once,
//     and its rows of the small operand from L2 (every workgroup reads all of the small
//     operand: M x K x 2 bytes each, which is why this pays only while M is small);
//   - an operand may be K-contiguous (a row of a stage is 256 contiguous bytes, two whole
//     cache lines) or contiguous along M or N, in which case a k row of the tile is 128
//     bytes (a 64-wide side: one whole cache line, what the large operand wants) or 64 (a
//     32-wide side: half the waste where the small operand has 16 rows), and the fragments
//     are transposed on the way to registers by ds_read_b64_tr_b16;
//   - a side may also be 16 wide (k rows of 32 bytes where the operand is contiguous along
//     M or N): a small operand of at most 16 rows then puts a quarter less through the
//     compute unit's load path than 32 rows, half of them zeros (16 x 4096 x 14336: 22.9 ->
//     19.9 us), and 16 rows of the LARGE operand per workgroup make 256 tiles of N = 4096, a
//     workgroup for every compute unit without any exchange between workgroups
//     (32 x 4096 x 14336: 22.6 -> 19.4 us);
//   - the LDS holds a ring of 3 to 6 stages of BK = 128 per workgroup (what fits 76 KB), two
//     workgroups to a compute unit (48..96 KB of loads in flight per compute unit: what it
//     takes to cover the latency of HBM at 20..40 GB/s per compute unit), filled by
//     buffer_load ... lds, 1 KiB per instruction (4 rows x 256 bytes);
//   - where the tile grid is one tile high, the panels start their walk along K at
//     staggered stages, so that the workgroups do not all ask the same memory channels at
//     the same time;
//   - the MFMAs are written out, accumulating in place: the compiler's own placement moved
//     the accumulators around every stage;
//   - the four waves split the K range of a stage (32 each) and every wave multiplies the
//     whole tile on v_mfma_f32_16x16x32; at the end the four partial tiles are added in
//     wave order through LDS and the sum is converted and stored;
//   - rows past M or N are read as zeros (the buffer descriptors end with the operand)
//     and not stored; so are the columns of a last stage past K (K a multiple of 8 where an
//     operand is K-contiguous, so that its rows stay 16-byte aligned);
//   - where the tiles are too few for the compute units (a 64-wide side on N = 8192 gives
//     128 of them), args.k_slices workgroups share a tile, each with a run of the stages:
//     every one writes its fp32 tile to args.partials, counts itself in at the tile's
//     counter, and the one that finds itself last adds the tiles up in slice order (so the
//     sum of an element is the same in every run, whoever is last), stores C and puts the
//     counter back to zero.  One launch still, and nobody waits for anybody.
//
// LDS layout of a stage: the A tile (BM rows), then the B tile (BN rows).  K-contiguous
// operand: a row is 16 chunks of 16 bytes, chunk c of row r in slot c ^ (r mod 16), so
// that the 16 rows a fragment read touches per k chunk fall on 16 different slots (all 64
// banks once).  M/N-contiguous operand: 128 k rows of 64, 32 or 16 elements; the 32-byte
// pieces of k row k are permuted within the row (mn_piece; 16 wide: the rows themselves,
// mn_row16), so that the 4 k rows x 32 bytes that 16 lanes of a transposing read touch, and
// those of the next 16 lanes 8 rows further on, fall on different banks (64 wide, in memory
// order, they are 4-way conflicts: 16 x 8192 x 8192 with B row-major 29.6 us, with the
// pieces permuted 28.1 us; B column-major, whose fragments are plain 16-byte reads, 24.3 us,
// at the time; the bank-conflict counter now reads the same for both kinds of kernel).
//
// Role with respect to the reference: as the other kernels, its gemm_impl (reference
// rocm_wmma_gemm/include/rocm_wmma_gemm/kernel/kernel.hpp:108-556); the reference has no
// kernel for these shapes and serves them with its nearest tuned tile (reference
// rocm_wmma_gemm/config/generate_config.py:174-234).
#ifndef ROCM_WMMA_GEMM_STREAM_KERNEL_HPP
#define ROCM_WMMA_GEMM_STREAM_KERNEL_HPP

#include "direct_kernel.hpp"

namespace rocm_wmma_gemm
{
namespace device
{

template<in_kind IN, class OutT, int BM, int BN, bool A_KMAJOR = true, bool B_KMAJOR = true>
struct stream_gemm
{
    using InT = typename std::conditional<IN == in_kind::f16, _Float16, __bf16>::type;

    static constexpr int BK        = 128;
    static constexpr int ROW_BYTES = BK * 2;
    static constexpr int WAVES     = 4;
    static constexpr int THREADS   = 64 * WAVES;
    static constexpr int A_BYTES   = BM * ROW_BYTES;
    static constexpr int B_BYTES   = BN * ROW_BYTES;
    static constexpr int STAGE     = A_BYTES + B_BYTES;
    // The ring: as many stages as fit 76 KB, at least 3 and at most 8, so that two workgroups
    // share a compute unit (all tiles but 64 x 64, whose three stages take 96 KB): while one
    // fills its ring or adds up and stores its tile, the other keeps the loads coming.
    // Against one workgroup per compute unit with a ring of 144 KB, same plans: +9.6 %
    // (geometric mean over 135 skinny problems), 16 x 28672 x 8192 4.1 -> 4.6 TB/s.  (A ring
    // of 112 or 152 KB is no better where a compute unit has one workgroup anyway: 128 tiles of
    // 16 x 8192 x 8192, 21.4 us with 3 stages of 32 x 64, 21.3 and 21.7 us with 4 and 6.  Nor
    // is reading the fragments of stage t + 1 under the MFMAs of stage t: it asks for a stage
    // one stage earlier, 21.5 -> 26.7 us.)
    static constexpr int RING_KB   = 76;
    static constexpr int DEPTH_FIT = (RING_KB * 1024) / STAGE < 3 ? 3 : (RING_KB * 1024) / STAGE;
    static constexpr int DEPTH     = DEPTH_FIT < 8 ? DEPTH_FIT : 8;
    static constexpr int LDS_BYTES = DEPTH * STAGE;
    static constexpr int TM        = BM / 16; // MFMA tiles of a workgroup tile
    static constexpr int TN        = BN / 16;
    // 1 KiB loads (4 rows) of a stage per wave: load q of an operand covers rows 4q .. 4q+3
    // and belongs to wave q mod 4
    // (M/N-contiguous, W wide: load q covers the 512 / W k rows from (512 / W) q on, W / 4
    // loads a stage)
    static constexpr int LOADS_A = BM / 16;
    static constexpr int LOADS_B = BN / 16;
    static constexpr int PER     = LOADS_A + LOADS_B;
    static constexpr int MAX_SLICES = 8; // workgroups that may share a tile (args.k_slices)
    static_assert((BM == 16 || BM == 32 || BM == 64 || BM == 128) && (BN == 16 || BN == 32 || BN == 64 || BN == 128)
                      && BM + BN >= 48 && BM + BN <= 192,
                  "tiles of 16, 32, 64 or 128 rows and columns, three stages of which fit the LDS");
    static_assert(LDS_BYTES <= 160 * 1024, "the ring must fit the 160 KB LDS");
    static_assert(DEPTH >= 3 && (DEPTH - 1) * PER < 64, "ring depth against the 6-bit vmcnt");
    static_assert(WAVES * BM * BN * 4 <= LDS_BYTES, "the partial tiles of the waves reuse the ring");

    // s_waitcnt immediate: vmcnt(n), lgkmcnt and expcnt untouched
    static constexpr int vmcnt_imm(int n)
    {
        return (n & 15) | (7 << 4) | (15 << 8) | ((n >> 4) << 14);
    }

    __device__ __forceinline__ static u32x4 descriptor(const InT* origin, long long bytes)
    {
        const unsigned long long p = (unsigned long long)origin;
        const unsigned int       lo = __builtin_amdgcn_readfirstlane((unsigned int)p);
        const unsigned int       hi = __builtin_amdgcn_readfirstlane((unsigned int)(p >> 32));
        const unsigned int       records
            = __builtin_amdgcn_readfirstlane(bytes <= 0 ? 0u : bytes > 0x7fffffffll ? 0x7fffffffu : (unsigned int)bytes);
        return u32x4{lo, hi & 0xffffu, records, 0x00020000u};
    }

    // One 1 KiB load: lane l's 16 bytes go to lds_block + 16 l.  (The compiler does not
    // look for hazards around inline assembly: four wait states cover M0 and a descriptor
    // or offset that a v_readfirstlane has just written.)
    // ONCE: with the non-temporal hint (gemm_args::stream_once).
    template<bool ONCE>
    __device__ __forceinline__ static void load_block(unsigned int lds_block, unsigned int voff, const u32x4& rsrc,
                                                      unsigned int soff)
    {
        if constexpr(ONCE)
        {
            asm volatile("s_mov_b32 m0, %[ldsb]\n\t"
                         "s_nop 4\n\t"
                         "buffer_load_dwordx4 %[voff], %[rsrc], %[soff] offen nt lds"
                         :
                         : [ldsb] "s"(lds_block), [voff] "v"(voff), [rsrc] "s"(rsrc), [soff] "s"(soff)
                         : "memory");
        }
        else
        {
            asm volatile("s_mov_b32 m0, %[ldsb]\n\t"
                         "s_nop 4\n\t"
                         "buffer_load_dwordx4 %[voff], %[rsrc], %[soff] offen lds"
                         :
                         : [ldsb] "s"(lds_block), [voff] "v"(voff), [rsrc] "s"(rsrc), [soff] "s"(soff)
                         : "memory");
        }
    }

    // M/N-contiguous operand, W elements wide (a k row of 2 W bytes; 512 / W k rows per 1 KiB
    // load).  Where the 32-byte pieces of k row k lie within the row: piece j in place
    // j ^ mn_piece(k).  A transposing read touches, per 16 lanes, 32 bytes of 4 consecutive
    // k rows, and the next 16 lanes the same 8 rows further on: W = 64, rows 128 bytes apart,
    // rows k and k + 2 and the rows 8 further all start on the same bank; W = 32, rows k and
    // k + 4 do (the 4 rows of a group do not meet), and the rows 8 further.
    // W = 128, rows 256 bytes apart: the 4 rows of a group all start on the same bank, so
    // each goes to another 32-byte place (k mod 4), and the rows 8 further on 128 bytes off.
    template<int W>
    __device__ __forceinline__ static int mn_piece(int k)
    {
        return W == 128 ? ((k & 3) ^ (((k >> 3) & 1) << 2)) : W == 64 ? ((k & 3) ^ ((k >> 3) & 1)) : ((k >> 3) & 1);
    }

    // W = 16: k rows of 32 bytes, 32 of them per 1 KiB load.  The 4 rows that 16 lanes of a
    // transposing read touch are 128 contiguous bytes, and the next 16 lanes' rows, 8 further
    // on, would start 256 bytes later on the same banks: of every second run of 8 rows the
    // two halves change places (row r of a wave's 32 lies in place r ^ 4 when r / 8 is odd),
    // so that one group reads the low 128 bytes of its 256 and the next the high.
    __device__ __forceinline__ static int mn_row16(int r)
    {
        return r ^ (((r >> 3) & 1) << 2);
    }

    // byte offset of lane l's 16 bytes of load `wave` (+ 4 i) from the operand's stage origin
    template<int W>
    __device__ __forceinline__ static unsigned int mn_load_offset(int lane, int wave, long long ld)
    {
        constexpr int LANES_PER_ROW = W / 8, ROWS_PER_LOAD = 512 / W;
        if constexpr(W == 16)
        {
            // a k row is one 32-byte piece: the rows change places instead (mn_row16)
            return (unsigned int)(((32 * wave + mn_row16(lane >> 1)) * ld + (lane & 1) * 8) * 2);
        }
        const int     k      = ROWS_PER_LOAD * wave + lane / LANES_PER_ROW; // (mod 16 as for every i)
        const int     place  = (lane % LANES_PER_ROW) >> 1;
        const int     piece  = place ^ mn_piece<W>(k);
        return (unsigned int)((k * ld + piece * 16 + (lane & 1) * 8) * 2);
    }

    // LDS offset, within the operand's part of a stage, of what lane (sub, slot) addresses for
    // column piece 0 of its transposing reads
    template<int W>
    __device__ __forceinline__ static int mn_read_offset(int wave, int sub, int slot)
    {
        if constexpr(W == 16)
        {
            return (32 * wave + mn_row16(8 * sub + (slot >> 2))) * 32 + (slot & 3) * 8;
        }
        const int k = 32 * wave + 8 * sub + (slot >> 2);
        return k * (2 * W) + mn_piece<W>(k) * 32 + (slot & 3) * 8;
    }

    // The fragments of a 64-wide side: column piece j of this lane's rows lies at addr ^ 32 j
    // (the stage and the rows are whole multiples of 128 bytes), the 4 rows further on 512
    // bytes later.  (One statement for the four fragments, with its own wait: the compiler
    // does not know that these registers are filled later, and would copy them into place at
    // once; four separate statements would be four trips to LDS in a row.)
    __device__ __forceinline__ static void transposed(unsigned int addr, u32x4 (&f)[4])
    {
        const unsigned int a1 = addr ^ 32u, a2 = addr ^ 64u, a3 = addr ^ 96u;
        uint2              l0, h0, l1, h1, l2, h2, l3, h3;
        asm volatile("ds_read_b64_tr_b16 %0, %8\n\t"
                     "ds_read_b64_tr_b16 %1, %8 offset:512\n\t"
                     "ds_read_b64_tr_b16 %2, %9\n\t"
                     "ds_read_b64_tr_b16 %3, %9 offset:512\n\t"
                     "ds_read_b64_tr_b16 %4, %10\n\t"
                     "ds_read_b64_tr_b16 %5, %10 offset:512\n\t"
                     "ds_read_b64_tr_b16 %6, %11\n\t"
                     "ds_read_b64_tr_b16 %7, %11 offset:512\n\t"
                     "s_waitcnt lgkmcnt(0)"
                     : "=&v"(l0), "=&v"(h0), "=&v"(l1), "=&v"(h1), "=&v"(l2), "=&v"(h2), "=&v"(l3), "=&v"(h3)
                     : "v"(addr), "v"(a1), "v"(a2), "v"(a3)
                     : "memory");
        f[0] = u32x4{l0.x, l0.y, h0.x, h0.y};
        f[1] = u32x4{l1.x, l1.y, h1.x, h1.y};
        f[2] = u32x4{l2.x, l2.y, h2.x, h2.y};
        f[3] = u32x4{l3.x, l3.y, h3.x, h3.y};
    }

    // a 128-wide side: rows of 256 bytes, eight column pieces, the 4 rows further on 1024
    // bytes later (two statements of four pieces: sixteen results in one would hold 32
    // registers early-clobbered at once)
    __device__ __forceinline__ static void transposed(unsigned int addr, u32x4 (&f)[8])
    {
#pragma unroll
        for(int h = 0; h < 2; ++h)
        {
            const unsigned int a0 = addr ^ (128u * h), a1 = a0 ^ 32u, a2 = a0 ^ 64u, a3 = a0 ^ 96u;
            uint2              l0, h0, l1, h1, l2, h2, l3, h3;
            asm volatile("ds_read_b64_tr_b16 %0, %8\n\t"
                         "ds_read_b64_tr_b16 %1, %8 offset:1024\n\t"
                         "ds_read_b64_tr_b16 %2, %9\n\t"
                         "ds_read_b64_tr_b16 %3, %9 offset:1024\n\t"
                         "ds_read_b64_tr_b16 %4, %10\n\t"
                         "ds_read_b64_tr_b16 %5, %10 offset:1024\n\t"
                         "ds_read_b64_tr_b16 %6, %11\n\t"
                         "ds_read_b64_tr_b16 %7, %11 offset:1024\n\t"
                         "s_waitcnt lgkmcnt(0)"
                         : "=&v"(l0), "=&v"(h0), "=&v"(l1), "=&v"(h1), "=&v"(l2), "=&v"(h2), "=&v"(l3), "=&v"(h3)
                         : "v"(a0), "v"(a1), "v"(a2), "v"(a3)
                         : "memory");
            f[4 * h + 0] = u32x4{l0.x, l0.y, h0.x, h0.y};
            f[4 * h + 1] = u32x4{l1.x, l1.y, h1.x, h1.y};
            f[4 * h + 2] = u32x4{l2.x, l2.y, h2.x, h2.y};
            f[4 * h + 3] = u32x4{l3.x, l3.y, h3.x, h3.y};
        }
    }

    // a 32-wide side: rows of 64 bytes, two column pieces
    __device__ __forceinline__ static void transposed(unsigned int addr, u32x4 (&f)[2])
    {
        const unsigned int a1 = addr ^ 32u;
        uint2              l0, h0, l1, h1;
        asm volatile("ds_read_b64_tr_b16 %0, %4\n\t"
                     "ds_read_b64_tr_b16 %1, %4 offset:256\n\t"
                     "ds_read_b64_tr_b16 %2, %5\n\t"
                     "ds_read_b64_tr_b16 %3, %5 offset:256\n\t"
                     "s_waitcnt lgkmcnt(0)"
                     : "=&v"(l0), "=&v"(h0), "=&v"(l1), "=&v"(h1)
                     : "v"(addr), "v"(a1)
                     : "memory");
        f[0] = u32x4{l0.x, l0.y, h0.x, h0.y};
        f[1] = u32x4{l1.x, l1.y, h1.x, h1.y};
    }

    // a 16-wide side: rows of 32 bytes, one column piece; the 4 rows further on lie 128 bytes
    // up or down (mn_row16): at addr ^ 128
    __device__ __forceinline__ static void transposed(unsigned int addr, u32x4 (&f)[1])
    {
        const unsigned int a1 = addr ^ 128u;
        uint2              l0, h0;
        asm volatile("ds_read_b64_tr_b16 %0, %2\n\t"
                     "ds_read_b64_tr_b16 %1, %3\n\t"
                     "s_waitcnt lgkmcnt(0)"
                     : "=&v"(l0), "=&v"(h0)
                     : "v"(addr), "v"(a1)
                     : "memory");
        f[0] = u32x4{l0.x, l0.y, h0.x, h0.y};
    }

    // acc += A fragment x B fragment, in place.  (Written out: left to place the
    // accumulators itself, the compiler moved them to other registers and back around every
    // stage, up to 50 moves a stage in the kernels with transposing reads: 16 x 8192 x 8192
    // with neither operand K-contiguous 26.1 - 32.9 us against 22.8 us, B row-major 28.4 against
    // 22.9, both K-contiguous 24.5 against 23.9; the 64 x 64 tile 35.4 against 27.2.)
    __device__ __forceinline__ static void multiply_add(f32x4& acc, const u32x4& fa, const u32x4& fb)
    {
        if constexpr(IN == in_kind::f16)
        {
            asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(fa), "v"(fb));
        }
        else
        {
            asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(fa), "v"(fb));
        }
    }

    // The compiler does not see that multiply_add reads and writes the accumulators on the
    // matrix pipeline: this keeps the wait states between its own writes (the zeros) and the
    // first multiply_add, and between the last multiply_add and its own reads.
    __device__ __forceinline__ static void settle(f32x4 (&acc)[TM][TN])
    {
#pragma unroll
        for(int i = 0; i < TM; ++i)
        {
#pragma unroll
            for(int j = 0; j < TN; ++j)
            {
                asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 3" : "+a"(acc[i][j]));
            }
        }
    }

    __device__ __forceinline__ static void run(const gemm_args& args)
    {
        __shared__ __attribute__((aligned(1024))) char lds_raw[LDS_BYTES];
        lds_char_ptr       lds      = (lds_char_ptr)lds_raw;
        const unsigned int lds_addr = (unsigned int)(size_t)lds;

        const int lane = threadIdx.x & 63;
        const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

        // Tile of this workgroup.  Workgroup ids that are congruent mod 8 run on the same
        // XCD; when the tile grid has two or more tiles along its short side, the
        // workgroups that share a panel of the large operand are given ids 8 apart, so
        // that the panel crosses the fabric once and the others find it in that XCD's L2.
        const int tiles = args.grid_m * args.grid_n;
        const int slice = blockIdx.x / tiles; // (slices outermost: the tile's place on its XCD stays)
        const int wg    = blockIdx.x - slice * tiles;
        int       tm, tn;
        if(args.grid_m <= args.grid_n && args.grid_n % 8 == 0)
        {
            const int xcd = wg & 7, j = wg >> 3;
            tm = j % args.grid_m;
            tn = (j / args.grid_m) * 8 + xcd;
        }
        else if(args.grid_n < args.grid_m && args.grid_m % 8 == 0)
        {
            const int xcd = wg & 7, j = wg >> 3;
            tn = j % args.grid_n;
            tm = (j / args.grid_n) * 8 + xcd;
        }
        else
        {
            tm = wg % args.grid_m;
            tn = wg / args.grid_m;
        }
        const long long batch = blockIdx.y;
        const int       row0 = tm * BM, col0 = tn * BN;
        const long long lda = args.lda, ldb = args.ldb;
        // K-contiguous: rows of the tile are rows of the operand, and the descriptor ends
        // with the rows of this batch entry, so a tile that hangs over the edge reads zeros
        // there.  M/N-contiguous: the tile is 64 columns of the operand's K rows, the
        // descriptor ends with the batch entry, and columns past the edge read what lies
        // there (the next k row): they only reach columns of C that are not stored.
        const InT* a0 = static_cast<const InT*>(args.A) + batch * args.batch_stride_a
                        + (A_KMAJOR ? (long long)row0 * lda : (long long)row0);
        const InT* b0 = static_cast<const InT*>(args.B) + batch * args.batch_stride_b
                        + (B_KMAJOR ? (long long)col0 * ldb : (long long)col0);
        const u32x4 rsrc_a = descriptor(a0, A_KMAJOR ? (long long)(args.M - row0) * lda * 2
                                                     : ((long long)args.K * lda - row0) * 2);
        const u32x4 rsrc_b = descriptor(b0, B_KMAJOR ? (long long)(args.N - col0) * ldb * 2
                                                     : ((long long)args.K * ldb - col0) * 2);

        // K-contiguous: load q = wave + 4 i of an operand covers rows 4q + l/16, LDS slot
        // l%16 of that row, so the lane fetches chunk (l%16) ^ (row mod 16), and row mod 16 =
        // 4 wave + l/16 for every i.  M/N-contiguous, W wide: a k row is 2 W bytes, load
        // q = wave + 4 i covers the 512 / W k rows from (512 / W) q on, and the lane fills
        // 16-byte slot l mod (W / 8) of its row, which holds the half l%2 of the 32-byte piece
        // that mn_piece() puts there.
        const int          sub    = lane >> 4, slot = lane & 15;
        const int          chunk  = slot ^ ((4 * wave + sub) & 15);
        const unsigned int voff_a = A_KMAJOR ? (unsigned int)(((4 * wave + sub) * lda + chunk * 8) * 2)
                                             : mn_load_offset<BM>(lane, wave, lda);
        const unsigned int voff_b = B_KMAJOR ? (unsigned int)(((4 * wave + sub) * ldb + chunk * 8) * 2)
                                             : mn_load_offset<BN>(lane, wave, ldb);
        // bytes from load i to load i+1 (16 rows, or 4 loads' worth of k rows), and from stage
        // to stage
        // (a 16-wide side has one load per wave and stage, and no step)
        const unsigned int step_a  = (unsigned int)((A_KMAJOR ? 16 : 4 * (512 / BM)) * lda * 2);
        const unsigned int step_b  = (unsigned int)((B_KMAJOR ? 16 : 4 * (512 / BN)) * ldb * 2);
        const unsigned int stage_a = A_KMAJOR ? (unsigned int)ROW_BYTES : (unsigned int)(BK * lda * 2);
        const unsigned int stage_b = B_KMAJOR ? (unsigned int)ROW_BYTES : (unsigned int)(BK * ldb * 2);

        // this workgroup's run of the K / BK stages
        // (K need not be whole stages: of a last stage that K cuts short, the lanes of a
        // K-contiguous operand whose 8 columns lie past K load out of range and get zeros;
        // the k rows of an M/N-contiguous operand past K lie past the end of its descriptor)
        const int          k_tail     = args.K % BK;
        const unsigned int past_range = 0x80000000u;
        const unsigned int voff_a_tail = A_KMAJOR && k_tail != 0 && chunk * 8 >= k_tail ? past_range : voff_a;
        const unsigned int voff_b_tail = B_KMAJOR && k_tail != 0 && chunk * 8 >= k_tail ? past_range : voff_b;
        const int stages_all = (args.K + BK - 1) / BK, stages_per = (stages_all + args.k_slices - 1) / args.k_slices;
        const int first      = slice * stages_per;
        const int stages     = stages_all - first < stages_per ? stages_all - first : stages_per; // >= 1 (host)
        // (the hints are template arguments: the walk over the stages below exists in four
        // copies, one test per launch picks one; a test per load, two branches each, cost a
        // third of the time of a 64 x 64 stage)
        auto issue_as = [&](int stage, int slot_index, auto once_a, auto once_b) {
            const unsigned int base = lds_addr + slot_index * STAGE + wave * 1024;
            const bool         last = first + stage == stages_all - 1; // the stage that K may cut short
            const unsigned int va = last ? voff_a_tail : voff_a, vb = last ? voff_b_tail : voff_b;
#pragma unroll
            for(int i = 0; i < LOADS_A; ++i)
            {
                load_block<decltype(once_a)::value>(
                    base + i * 4096, va, rsrc_a,
                    __builtin_amdgcn_readfirstlane((unsigned int)(first + stage) * stage_a + i * step_a));
            }
#pragma unroll
            for(int i = 0; i < LOADS_B; ++i)
            {
                load_block<decltype(once_b)::value>(
                    base + A_BYTES + i * 4096, vb, rsrc_b,
                    __builtin_amdgcn_readfirstlane((unsigned int)(first + stage) * stage_b + i * step_b));
            }
        };
        // Where the tile grid is one tile high (a skinny M or N: no two workgroups read the
        // same panel of the large operand), every panel starts its run of stages at a
        // different place and wraps around.  Workgroups that walk K in step all ask for the
        // same 256 bytes of their rows at the same time, rows a power of two apart, and
        // those requests crowd onto a few memory channels: 16 x 8192 x 8192 with B
        // column-major 24.1 -> 21.0 us, 16 x 28672 x 8192 (470 MB of B, past the memory-side
        // cache) 100 -> 83 us.  (With two tiles to a panel, 128 x 8192 x 8192, the pair shares
        // the panel through L2 only while it walks in step, and staggering the panels gains
        // nothing there; staggering by XCD only is worse than not at all.)  The order of
        // the sum of an element depends on its tile's place alone: results stay the same
        // from run to run.
        const bool one_high = args.grid_m == 1 || args.grid_n == 1;
        const int  panel = args.grid_m <= args.grid_n ? tn : tm, panels = args.grid_m <= args.grid_n ? args.grid_n : args.grid_m;
        const int  turn  = one_high ? (int)(((long long)panel * stages) / panels) : 0;
        // Past the last stage the loads fetch the last stage again into slots that nobody
        // reads any more: the number of loads in flight stays what the waits assume.
        auto clamped = [&](int stage) {
            const int at = (stage < stages ? stage : stages - 1) + turn;
            return at >= stages ? at - stages : at;
        };

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
        settle(acc);

        // fragment of this wave's K step (k 32 wave .. 32 wave + 31 of the stage).
        // K-contiguous: row l%16 of a 16-row block, k chunk 4 wave + l/16.  M/N-contiguous:
        // two transposing reads of 4 k rows x 16 elements per 16 lanes; lane p of a group of
        // 16 supplies the address of 4 elements of k row p/4 (ds_read_b64_tr_b16 hands lane
        // i, element j what lane 4j + i/4 addressed, element i%4), so the group that feeds k
        // 8 g .. 8 g + 7 reads rows 32 wave + 8 g + p/4 and the same 4 rows further on.
        const int frag_off = slot * ROW_BYTES + (((4 * wave + sub) ^ slot) & 15) * 16;
        const int tr_off_a = mn_read_offset<BM>(wave, sub, slot);
        const int tr_off_b = mn_read_offset<BN>(wave, sub, slot);
        using lds_u32x4    = __attribute__((address_space(3))) u32x4;

        // (The accumulators enter and leave a copy of the walk through settle(): where the
        // copies meet again the compiler may move them between registers, and it does not know
        // that the multiply_adds before such a move are still on the matrix pipeline.)
        auto walk = [&](auto once_a, auto once_b) {
        auto issue = [&](int stage, int slot) { issue_as(stage, slot, once_a, once_b); };
        for(int t = 0; t < DEPTH - 1; ++t)
        {
            issue(clamped(t), t);
        }
        settle(acc);
        int slot_index = 0; // of stage t
        for(int t = 0; t < stages; ++t)
        {
            // stage t has landed (the loads of the DEPTH - 2 stages after it may be in
            // flight), in every wave: then its slot may be read, and the slot of stage
            // t - 1, which every wave has finished reading, may be filled again
            __builtin_amdgcn_s_waitcnt(vmcnt_imm((DEPTH - 2) * PER));
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            issue(clamped(t + DEPTH - 1), slot_index == 0 ? DEPTH - 1 : slot_index - 1);

            lds_char_ptr       sa   = lds + slot_index * STAGE + frag_off;
            const unsigned int sa_t = lds_addr + slot_index * STAGE;
            u32x4              fa[TM], fb[TN];
            if constexpr(A_KMAJOR)
            {
#pragma unroll
                for(int i = 0; i < TM; ++i)
                {
                    fa[i] = *reinterpret_cast<lds_u32x4*>(sa + i * 16 * ROW_BYTES);
                }
            }
            else
            {
                transposed(sa_t + tr_off_a, fa);
            }
            if constexpr(B_KMAJOR)
            {
#pragma unroll
                for(int j = 0; j < TN; ++j)
                {
                    fb[j] = *reinterpret_cast<lds_u32x4*>(sa + A_BYTES + j * 16 * ROW_BYTES);
                }
            }
            else
            {
                transposed(sa_t + A_BYTES + tr_off_b, fb);
            }
#pragma unroll
            for(int i = 0; i < TM; ++i)
            {
#pragma unroll
                for(int j = 0; j < TN; ++j)
                {
                    multiply_add(acc[i][j], fa[i], fb[j]);
                }
            }
            slot_index = slot_index + 1 == DEPTH ? 0 : slot_index + 1;
        }
        settle(acc);
        };
        const int once = __builtin_amdgcn_readfirstlane(args.stream_once);
        if(once == 0)
        {
            walk(std::false_type{}, std::false_type{});
        }
        else if(once == 1)
        {
            walk(std::false_type{}, std::true_type{});
        }
        else if(once == 2)
        {
            walk(std::true_type{}, std::false_type{});
        }
        else
        {
            walk(std::true_type{}, std::true_type{});
        }

        // every load has landed and every wave has read its last stage: the ring becomes
        // the four partial tiles, [wave][BM][BN] fp32
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        settle(acc);
        using lds_float = __attribute__((address_space(3))) float;
        lds_float* part = reinterpret_cast<lds_float*>(lds);
#pragma unroll
        for(int i = 0; i < TM; ++i)
        {
#pragma unroll
            for(int j = 0; j < TN; ++j)
            {
#pragma unroll
                for(int v = 0; v < 4; ++v)
                {
                    // result register v of a 16 x 16 tile: row 4 (l/16) + v, column l%16
                    part[(wave * BM + 16 * i + 4 * sub + v) * BN + 16 * j + slot] = acc[i][j][v];
                }
            }
        }
        __syncthreads();
        OutT* C = static_cast<OutT*>(args.C) + batch * args.batch_stride_c;
        // (wave order: the sum of an element is the same in every run)
        auto tile_sum = [&](int e) {
            return ((part[e] + part[BM * BN + e]) + part[2 * BM * BN + e]) + part[3 * BM * BN + e];
        };
        auto store = [&](int e, float s) {
            const int row = e / BN, col = e % BN;
            if(row0 + row < args.M && col0 + col < args.N)
            {
                C[(long long)(row0 + row) * args.N + col0 + col] = to_out<OutT>(s);
            }
        };
        if(args.k_slices == 1)
        {
            for(int e = threadIdx.x; e < BM * BN; e += THREADS)
            {
                store(e, tile_sum(e));
            }
            return;
        }
        // Several workgroups per tile.  The tiles they exchange travel through memory that
        // every XCD sees the same way: stores and loads at device scope (sc1), which write
        // through, and miss in, the XCD's own L2; 16 bytes a lane.  A workgroup counts itself
        // in when its stores have been acknowledged, and reads the others' tiles only after
        // it has seen all of them counted, so nobody reads a piece that is half written.
        constexpr int   DEVICE_SCOPE = 16; // cache policy operand of the buffer builtins: sc1
        constexpr int   TILE4        = BM * BN / 4;
        const long long tile_lin     = batch * tiles + wg;
        const __amdgpu_buffer_rsrc_t shared = __builtin_amdgcn_make_buffer_rsrc(
            args.partials + tile_lin * args.k_slices * (long long)(BM * BN), 0, args.k_slices * BM * BN * 4, 0x00020000);
        using lds_f32x4 = __attribute__((address_space(3))) f32x4;
        for(int e4 = threadIdx.x; e4 < TILE4; e4 += THREADS)
        {
            const lds_f32x4* p4 = reinterpret_cast<const lds_f32x4*>(part) + e4;
            const f32x4      s  = ((p4[0] + p4[TILE4]) + p4[2 * TILE4]) + p4[3 * TILE4]; // (wave order)
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, s), shared, (slice * TILE4 + e4) * 16, 0,
                                                   DEVICE_SCOPE);
        }
        // (the stores above write through to memory and are acknowledged from there; a
        // release fence at device scope would write the whole L2 back instead, which costs
        // more than the GEMM)
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
        __syncthreads();
        __shared__ unsigned int arrived_before;
        if(threadIdx.x == 0)
        {
            // the counter holds (epoch << 8 | arrivals); a count under another launch's epoch
            // (something a killed kernel left behind) starts from zero
            unsigned int seen = __hip_atomic_load(args.arrivals + tile_lin, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            for(;;)
            {
                const unsigned int count = (seen >> 8) == args.arrival_epoch ? (seen & 255u) : 0u;
                if(__hip_atomic_compare_exchange_strong(args.arrivals + tile_lin, &seen,
                                                        (args.arrival_epoch << 8) | (count + 1u), __ATOMIC_RELAXED,
                                                        __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
                {
                    arrived_before = count;
                    break;
                }
            }
        }
        __syncthreads();
        if(arrived_before != (unsigned int)(args.k_slices - 1))
        {
            return; // the last one to arrive finishes the tile
        }
        // (all slices' loads of a piece go out before the first is used: a loop over the
        // slices would pay a trip to memory per slice; the host keeps k_slices <= MAX_SLICES)
        for(int e4 = threadIdx.x; e4 < TILE4; e4 += THREADS)
        {
            f32x4 v[MAX_SLICES];
#pragma unroll
            for(int q = 0; q < MAX_SLICES; ++q)
            {
                v[q] = q < args.k_slices
                           ? __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(shared, (q * TILE4 + e4) * 16,
                                                                                             0, DEVICE_SCOPE))
                           : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            }
            f32x4 s = v[0];
#pragma unroll
            for(int q = 1; q < MAX_SLICES; ++q)
            {
                s = q < args.k_slices ? s + v[q] : s;
            }
#pragma unroll
            for(int c = 0; c < 4; ++c)
            {
                store(4 * e4 + c, s[c]);
            }
        }
        if(threadIdx.x == 0)
        {
            // back to zero arrivals, for a replay of this launch (same epoch)
            __hip_atomic_store(args.arrivals + tile_lin, args.arrival_epoch << 8, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        }
    }
};

} // namespace device
} // namespace rocm_wmma_gemm

#endif // ROCM_WMMA_GEMM_STREAM_KERNEL_HPP
