// Register-staged MFMA GEMM kernel for gfx950 (wave64, v_mfma_f32_32x32x16).
//
// One workgroup computes a BM x BN tile of a ROW-MAJOR C over the whole K range
// (or over one K slice when split-K is on).  Column-major C is served by the host
// as the transposed problem, so no kernel here ever writes a column-major C.
//
// Data path per K step of BK:
//   global --(16-byte or 2-byte guarded loads)--> VGPRs --> LDS --> MFMA operands
// Both operand tiles live in LDS in the same K-contiguous form, whatever their
// layout in memory: row r of the tile is BK elements, stored as BK/8 chunks of
// 16 bytes, chunk c of row r at slot c ^ swizzle(r).  An operand that is
// contiguous along M or N in memory is transposed in registers (8x8 blocks of
// 16-bit elements) on its way to LDS, so its global loads stay 16 bytes wide and
// coalesced along the contiguous dimension.
//
// This kernel replaces the reference's gemm_impl / prefetch_fragment /
// load_matrix / store_matrix / load_shared_to_global chain (reference
// rocm_wmma_gemm/include/rocm_wmma_gemm/kernel/kernel.hpp:108-556,
// kernel/load.hpp:348-966, kernel/fragment.hpp:191-404) and its WMMA wrapper
// (kernel/wmma.hpp:44-85).  Unlike the reference it accumulates in fp32 for every
// type pair, guards M, N and K tails, and accepts odd leading dimensions.
#ifndef ROCM_WMMA_GEMM_GEMM_KERNEL_HPP
#define ROCM_WMMA_GEMM_GEMM_KERNEL_HPP

#include <hip/hip_runtime.h>

#include "tile_map.hpp"

namespace rocm_wmma_gemm
{
namespace device
{

using u32x4  = unsigned int __attribute__((ext_vector_type(4)));
using f16x8  = _Float16 __attribute__((ext_vector_type(8)));
using bf16x8 = __bf16 __attribute__((ext_vector_type(8)));
using f32x16 = float __attribute__((ext_vector_type(16)));
using f32x4  = float __attribute__((ext_vector_type(4)));

enum class in_kind
{
    f16  = 0,
    bf16 = 1
};

// How operand tiles are fetched from global memory.
enum class load_mode
{
    vec_unguarded = 0, // 16-byte loads, tile fully inside the matrix, K % BK == 0
    vec_guarded   = 1, // 16-byte loads, whole chunks zero-filled outside the matrix
    scalar        = 2 // 2-byte guarded loads: any leading dimension, any alignment
};

struct gemm_args
{
    void*       C;
    const void* A;
    const void* B;
    int         M, N, K; // C is M x N row-major in kernel space
    long long   lda, ldb; // leading dimension of each operand along its contiguous axis:
                          // K (or the padded K) if K-contiguous, else the row count
    long long   batch_stride_a, batch_stride_b, batch_stride_c; // elements
    int         grid_m, grid_n; // tiles along M and N
    int         group; // band height of the tile map (banded_tile): > 0 tile rows, < 0 tile columns
    int         k_slices; // split-K factor of the split tiles (1 = off)
    int         tail_begin; // tiles [0, tail_begin) of the walk order run whole K, the rest are
                            // split k_slices ways; 0 = every tile is split (plain split-K)
    float*      partials; // split-K workspace, fp32, or nullptr.  tail_begin == 0:
                          // [batch][slice][M][N] planes; else [batch][split tile][slice][BM][BN]
    int         blocks_per_batch; // workgroups' worth of work per batch entry (whole tiles + slices)
    int         batches; // batch entries of this launch; blocks_per_batch * batches fits an int
    int         stream_units; // persistent kernel only.  0: workgroups take whole items.  U > 0:
                              // workgroup g takes K tiles [g * U, (g + 1) * U) of the sequence of all
                              // K tiles of all tiles of all batch entries; partials then holds two
                              // [BM][BN] slots per workgroup
    int         k_tail; // persistent kernel with guarded stores only.  0: the operands hold K
                        // columns, a multiple of the K tile.  t > 0: they hold K - 64 + t
                        // columns, and the kernel reads zeros for the rest of the last K tile
    int         batch_by_xcd; // persistent and direct kernels, needs k_slices == 1 and
                              // blocks_per_batch * batches in an int.  1: the items (tile,
                              // batch entry) are dealt so that each XCD works through one
                              // contiguous run of batch entries, and the tiles of an entry, which
                              // share its A and B, go through one L2 at about the same time
    int         warm_ahead; // persistent kernel only.  1: beside the loads of a K tile, two waves
                            // of a workgroup touch a quarter of the cache lines of the K tile
                            // after it (one dword per line), so that the line is on its way into
                            // the XCD's L2 a tile time before the loads that need it; the
                            // workgroups that share an operand panel touch different quarters
    unsigned int* arrivals; // whole-K streaming kernel with k_slices > 1 only: one counter per
                            // tile and batch entry; partials then holds
                            // [batch][tile][slice][BM][BN]
    unsigned int  arrival_epoch; // this launch's tag in those counters (24 bits, not zero): a
                                 // counter holds (epoch << 8 | arrivals) and counts from zero
                                 // for a workgroup that finds another epoch in it
    int           k_block; // persistent kernel built with K_RUNS only.  b > 0 (a power of two): the K
                           // tiles of an item are walked in runs of b, and within every 8 runs the
                           // workgroups of XCD x take run x first and wrap round (solo_gemm::run
                           // says why); 0: in order
    int           k_group; // the same kernels.  g = 2, 4 or 8: within every aligned group of g K tiles
                           // the workgroup of tile (i, j) starts at tile (i + j) mod g of the group and
                           // wraps round, so that the workgroups of an XCD that share a panel ask for
                           // a line at different times and all but the first find it in L2; 0: in order
    int           stream_once; // streaming kernel.  Bit 0: B's loads carry the non-temporal hint, bit 1:
                               // A's.  For an operand that is read once and does not fit the 256 MB
                               // memory-side cache: its lines then take no room there that they cannot
                               // use, and the stream from HBM runs 15 % faster (7.1 against 6.1 TB/s
                               // for a kernel that only reads; 16 x 28672 x 8192 82 -> 76 us).  An
                               // operand that fits is better off without: back-to-back calls find it
                               // in that cache (16 x 8192 x 8192 20.6 us, 29 with the hint).
};

// What one workgroup works on.  blockIdx.x enumerates the whole tiles first, then
// (slice, split tile) pairs, slices outermost.
struct block_work
{
    int tile_id; // position in the tile walk (see map_tile)
    int slice, slices; // K slice of this workgroup and how many the tile has (1 = whole K)
};

__device__ __forceinline__ block_work decode_block(const gemm_args& args, int b)
{
    if(b < args.tail_begin || args.k_slices == 1)
    {
        return {b, 0, 1};
    }
    const int split_tiles = args.grid_m * args.grid_n - args.tail_begin;
    const int r           = b - args.tail_begin;
    const int slice       = r / split_tiles;
    return {args.tail_begin + (r - slice * split_tiles), slice, args.k_slices};
}

__device__ __forceinline__ block_work decode_block(const gemm_args& args)
{
    return decode_block(args, (int)blockIdx.x);
}

// Where a split workgroup's fp32 partial tile goes: a pointer P and a row pitch such
// that element (row, col) of C (global coordinates) is P[row * pitch + col].
template<int BM, int BN>
__device__ __forceinline__ float* partial_base(
    const gemm_args& args, const block_work& w, long long batch, int row0, int col0, long long& pitch)
{
    if(args.tail_begin == 0)
    {
        pitch = args.N;
        return args.partials + (batch * args.k_slices + w.slice) * (long long)args.M * args.N;
    }
    const long long split_tiles = args.grid_m * args.grid_n - args.tail_begin;
    const long long t           = w.tile_id - args.tail_begin;
    pitch                       = BN;
    return args.partials + ((batch * split_tiles + t) * args.k_slices + w.slice) * (long long)(BM * BN)
           - ((long long)row0 * BN + col0);
}

template<in_kind IN>
__device__ __forceinline__ f32x16 mfma_32x32x16(u32x4 a, u32x4 b, f32x16 c)
{
    if constexpr(IN == in_kind::f16)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(
            __builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    else
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(
            __builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
}

// 16x16x32: lane l feeds row (column) l%16, k 8*(l/16)..+7 of the first (second)
// operand; result register v is row 4*(l/16) + v, column l%16.
template<in_kind IN>
__device__ __forceinline__ f32x4 mfma_16x16x32(u32x4 a, u32x4 b, f32x4 c)
{
    if constexpr(IN == in_kind::f16)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(
            __builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    else
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            __builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
}

// fp32 -> C element, round to nearest even.
template<class OutT>
__device__ __forceinline__ OutT to_out(float v)
{
    return static_cast<OutT>(v);
}

// Chunk slot swizzle.  The LDS has 64 banks of 4 bytes (256 bytes per clock); a
// 16-byte-per-lane read of a wave is served in 4 cycles of 16 lanes each.  Measured
// on MI355X (two lanes alone on one bank column slow down iff they share a cycle): the
// cycles take, of each 32-lane half, the lanes of 4-lane quads {0,3,5,6} and
// {1,2,4,7}.  The 16 lanes of a cycle must hit 16 distinct 16-byte columns of a
// 256-byte line.  A row of CH chunks spans 16*CH bytes and 16/CH rows share a line.
//   * 32x32x16 MFMA (lane l reads row l%32, chunk l/32): a cycle reads one chunk of
//     rows 4q..4q+3 for the 4 quads q; slot = chunk ^ ((row / (16/CH)) % CH) gives
//     ~505 B/ns/CU, "chunk ^ (row % 8)" ~297 (two-way conflicts), no swizzle 76.
//   * 16x16x32 MFMA (lane l reads row l%16, chunk l/16): a cycle reads chunk g of
//     rows 0-3 and 12-15 and chunk g^1 of rows 4-11.  The slot above is conflict-free
//     for CH = 8 (~520 B/ns/CU) but two-way conflicted for CH = 4 (~300); there
//     slot = chunk ^ 2*((row / 8) % 2) separates the rows that share a line position.
template<int CH, int MI = 32>
__device__ __forceinline__ int swizzle_of_row(int row)
{
    static_assert(CH == 8 || CH == 4 || CH == 2, "unsupported BK");
    if constexpr(MI == 16 && CH == 4)
    {
        return 2 * ((row >> 3) & 1);
    }
    else
    {
        return (row * CH / 16) % CH;
    }
}

// 16-byte chunk index (in u32x4 units) of (row, chunk) inside a tile.
template<int CH>
__device__ __forceinline__ int lds_chunk_index(int row, int chunk)
{
    return row * CH + (chunk ^ swizzle_of_row<CH>(row));
}

// ---------------------------------------------------------------------------
// Global -> register staging of one operand tile.
//
// The tile is ROWS x BK in (row, k) space; element (row, k) of the operand sits at
// base[row * stride_row + k * stride_k], with (stride_row, stride_k) = (ld, 1) for a
// K-contiguous operand (KMAJOR) and (1, ld) otherwise.  Rows >= rows_left and
// k >= k_left read as zero.
// ---------------------------------------------------------------------------
template<bool KMAJOR, int ROWS, int BK, int THREADS, load_mode MODE>
struct operand_stage
{
    static constexpr int CH     = BK / 8; // 16-byte chunks per tile row
    static constexpr int CHUNKS = ROWS * CH; // chunks per tile
    static_assert(CHUNKS % THREADS == 0, "tile must divide evenly over the workgroup");
    static constexpr int PER_THREAD = CHUNKS / THREADS;

    // M/N-contiguous operands in vector mode are moved as 8(k) x VW(row) blocks.
    static constexpr int VW     = PER_THREAD >= 8 ? 8 : (PER_THREAD >= 4 ? 4 : (PER_THREAD >= 2 ? 2 : 1));
    static constexpr int BLOCKS = PER_THREAD / VW; // blocks per thread (transposed path)
    static constexpr bool TRANSPOSED = !KMAJOR && MODE != load_mode::scalar;
    static_assert(!TRANSPOSED || VW >= 2, "transposed path needs at least 2 chunks per thread");
    static_assert(!TRANSPOSED || ROWS % VW == 0, "rows must divide into blocks");

    // Data in flight.  KMAJOR/scalar: regs[i] is the finished LDS chunk i.
    // TRANSPOSED: regs[b*VW .. b*VW+VW) hold block b, already transposed by fetch().
    u32x4 regs[PER_THREAD];

    // --- chunk ownership -------------------------------------------------
    // K-contiguous / scalar K-contiguous: consecutive threads take consecutive
    // chunks of a row (coalesced along k).  Scalar M/N-contiguous: consecutive
    // threads take consecutive rows of the same chunk column (coalesced along row).
    __device__ __forceinline__ static void chunk_of(int i, int tid, int& row, int& chunk)
    {
        const int c = tid + i * THREADS;
        if constexpr(KMAJOR)
        {
            row   = c / CH;
            chunk = c % CH;
        }
        else
        {
            row   = c % ROWS;
            chunk = c / ROWS;
        }
    }
    // Transposed path: block b covers rows [rb*VW, rb*VW+VW) and chunk column kb.
    __device__ __forceinline__ static void block_of(int b, int tid, int& row0, int& chunk)
    {
        constexpr int ROW_BLOCKS = ROWS / VW;
        const int     c          = tid + b * THREADS;
        row0                     = (c % ROW_BLOCKS) * VW;
        chunk                    = c / ROW_BLOCKS;
    }

    template<class InT>
    __device__ __forceinline__ void fetch(const InT* __restrict__ base,
                                          long long               stride_row,
                                          long long               stride_k,
                                          int                     rows_left,
                                          int                     k_left,
                                          int                     tid)
    {
        if constexpr(MODE == load_mode::scalar)
        {
#pragma unroll
            for(int i = 0; i < PER_THREAD; ++i)
            {
                int row, chunk;
                chunk_of(i, tid, row, chunk);
                unsigned short e[8];
#pragma unroll
                for(int j = 0; j < 8; ++j)
                {
                    const int  k  = chunk * 8 + j;
                    const bool ok = row < rows_left && k < k_left;
                    const auto* p = reinterpret_cast<const unsigned short*>(base)
                                    + (ok ? row * stride_row + k * stride_k : 0);
                    const unsigned short v = *p;
                    e[j]                   = ok ? v : (unsigned short)0;
                }
                u32x4 r;
                r.x     = (unsigned)e[0] | ((unsigned)e[1] << 16);
                r.y     = (unsigned)e[2] | ((unsigned)e[3] << 16);
                r.z     = (unsigned)e[4] | ((unsigned)e[5] << 16);
                r.w     = (unsigned)e[6] | ((unsigned)e[7] << 16);
                regs[i] = r;
            }
        }
        else if constexpr(KMAJOR)
        {
#pragma unroll
            for(int i = 0; i < PER_THREAD; ++i)
            {
                int row, chunk;
                chunk_of(i, tid, row, chunk);
                const int k = chunk * 8;
                if constexpr(MODE == load_mode::vec_unguarded)
                {
                    regs[i] = *reinterpret_cast<const u32x4*>(base + row * stride_row + k);
                }
                else
                {
                    const bool ok = row < rows_left && k < k_left;
                    u32x4      v  = {0u, 0u, 0u, 0u};
                    if(ok)
                    {
                        v = *reinterpret_cast<const u32x4*>(base + row * stride_row + k);
                    }
                    regs[i] = v;
                }
            }
        }
        else
        {
            // 8 (k) x VW (row) block: VW*2-byte loads down 8 consecutive k, then an
            // in-register transpose so that each of the VW rows owns 8 consecutive k.
#pragma unroll
            for(int b = 0; b < BLOCKS; ++b)
            {
                int row0, chunk;
                block_of(b, tid, row0, chunk);
                unsigned int src[8][VW / 2]; // src[kk][pair of rows]
#pragma unroll
                for(int kk = 0; kk < 8; ++kk)
                {
                    const int  k = chunk * 8 + kk;
                    const bool ok
                        = MODE == load_mode::vec_unguarded || (row0 < rows_left && k < k_left);
                    const InT* p = base + (ok ? k * stride_k + row0 : 0);
                    if constexpr(VW == 8)
                    {
                        u32x4 v = *reinterpret_cast<const u32x4*>(p);
                        src[kk][0] = ok ? v.x : 0u;
                        src[kk][1] = ok ? v.y : 0u;
                        src[kk][2] = ok ? v.z : 0u;
                        src[kk][3] = ok ? v.w : 0u;
                    }
                    else if constexpr(VW == 4)
                    {
                        uint2 v    = *reinterpret_cast<const uint2*>(p);
                        src[kk][0] = ok ? v.x : 0u;
                        src[kk][1] = ok ? v.y : 0u;
                    }
                    else
                    {
                        unsigned int v = *reinterpret_cast<const unsigned int*>(p);
                        src[kk][0]     = ok ? v : 0u;
                    }
                }
#pragma unroll
                for(int r = 0; r < VW; ++r)
                {
                    // row r of the block takes half (r & 1) of dword r/2 from each k.
                    const unsigned sel = (r & 1) ? 0x07060302u : 0x05040100u;
                    u32x4          out;
                    out.x = __builtin_amdgcn_perm(src[1][r / 2], src[0][r / 2], sel);
                    out.y = __builtin_amdgcn_perm(src[3][r / 2], src[2][r / 2], sel);
                    out.z = __builtin_amdgcn_perm(src[5][r / 2], src[4][r / 2], sel);
                    out.w = __builtin_amdgcn_perm(src[7][r / 2], src[6][r / 2], sel);
                    regs[b * VW + r] = out;
                }
            }
        }
    }

    __device__ __forceinline__ void commit(u32x4* __restrict__ tile, int tid) const
    {
        if constexpr(TRANSPOSED)
        {
#pragma unroll
            for(int b = 0; b < BLOCKS; ++b)
            {
                int row0, chunk;
                block_of(b, tid, row0, chunk);
#pragma unroll
                for(int r = 0; r < VW; ++r)
                {
                    tile[lds_chunk_index<CH>(row0 + r, chunk)] = regs[b * VW + r];
                }
            }
        }
        else
        {
#pragma unroll
            for(int i = 0; i < PER_THREAD; ++i)
            {
                int row, chunk;
                chunk_of(i, tid, row, chunk);
                tile[lds_chunk_index<CH>(row, chunk)] = regs[i];
            }
        }
    }
};

// ---------------------------------------------------------------------------
// The kernel
// ---------------------------------------------------------------------------
template<in_kind IN,
         class OutT,
         bool      A_KMAJOR,
         bool      B_KMAJOR,
         int       BM,
         int       BN,
         int       BK,
         int       WAVES_M,
         int       WAVES_N,
         load_mode MODE>
struct staged_gemm
{
    using InT = typename std::conditional<IN == in_kind::f16, _Float16, __bf16>::type;

    static constexpr int THREADS = 64 * WAVES_M * WAVES_N;
    static constexpr int WTM     = BM / WAVES_M; // rows per wave
    static constexpr int WTN     = BN / WAVES_N; // columns per wave
    static constexpr int TM      = WTM / 32; // MFMA tiles per wave along M
    static constexpr int TN      = WTN / 32;
    static constexpr int CH      = BK / 8;
    static constexpr int A_TILE  = BM * CH; // u32x4 units
    static constexpr int B_TILE  = BN * CH;
    static constexpr int STAGE   = A_TILE + B_TILE;
    static constexpr int LDS_BYTES = 2 * STAGE * 16;
    static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be built from 32x32 MFMA tiles");
    static_assert(BK % 16 == 0, "BK must hold whole MFMA K steps");
    static_assert(LDS_BYTES <= 160 * 1024, "tile does not fit the 160 KB LDS");

    using stage_a = operand_stage<A_KMAJOR, BM, BK, THREADS, MODE>;
    using stage_b = operand_stage<B_KMAJOR, BN, BK, THREADS, MODE>;

    __device__ __forceinline__ static void compute_stage(const u32x4* __restrict__ lds_a,
                                                         const u32x4* __restrict__ lds_b,
                                                         f32x16 (&acc)[TM][TN],
                                                         int row_in_wave_a,
                                                         int row_in_wave_b,
                                                         int lane_hi)
    {
#pragma unroll
        for(int kk = 0; kk < BK / 16; ++kk)
        {
            u32x4     a[TM], b[TN];
            const int chunk = kk * 2 + lane_hi;
#pragma unroll
            for(int i = 0; i < TM; ++i)
            {
                a[i] = lds_a[lds_chunk_index<CH>(row_in_wave_a + i * 32, chunk)];
            }
#pragma unroll
            for(int j = 0; j < TN; ++j)
            {
                b[j] = lds_b[lds_chunk_index<CH>(row_in_wave_b + j * 32, chunk)];
            }
#pragma unroll
            for(int i = 0; i < TM; ++i)
            {
#pragma unroll
                for(int j = 0; j < TN; ++j)
                {
                    acc[i][j] = mfma_32x32x16<IN>(a[i], b[j], acc[i][j]);
                }
            }
        }
    }

    __device__ __forceinline__ static void run(const gemm_args& args)
    {
        __shared__ u32x4 lds[2 * STAGE];

        const int tid     = threadIdx.x;
        const int lane    = tid & 63;
        const int wave    = tid >> 6;
        const int wave_m  = wave / WAVES_N;
        const int wave_n  = wave % WAVES_N;
        const int lane_lo = lane & 31;
        const int lane_hi = lane >> 5;

        // blockIdx.x enumerates tiles and K slices; blockIdx.y the batch entry.
        const block_work w = decode_block(args);
        const int slice    = w.slice;
        const tile_coord t = map_tile(w.tile_id, args.grid_m, args.grid_n, args.group);
        const int row0 = t.m * BM;
        const int col0 = t.n * BN;

        // K range of this slice, in whole BK steps.
        const int k_steps_total = (args.K + BK - 1) / BK;
        const int steps_per     = (k_steps_total + w.slices - 1) / w.slices;
        const int step_begin    = slice * steps_per;
        int       step_end      = step_begin + steps_per;
        if(step_end > k_steps_total)
        {
            step_end = k_steps_total;
        }

        const long long batch = blockIdx.y;
        const InT* A = static_cast<const InT*>(args.A) + batch * args.batch_stride_a;
        const InT* B = static_cast<const InT*>(args.B) + batch * args.batch_stride_b;

        // Element (row, k) of A at A[row*a_sr + k*a_sk]; element (k, col) of B at B[col*b_sr + k*b_sk].
        const long long a_sr = A_KMAJOR ? args.lda : 1;
        const long long a_sk = A_KMAJOR ? 1 : args.lda;
        const long long b_sr = B_KMAJOR ? args.ldb : 1;
        const long long b_sk = B_KMAJOR ? 1 : args.ldb;

        const InT* a_tile = A + row0 * a_sr;
        const InT* b_tile = B + col0 * b_sr;
        const int  rows_a = args.M - row0;
        const int  rows_b = args.N - col0;

        f32x16 acc[TM][TN];
#pragma unroll
        for(int i = 0; i < TM; ++i)
        {
#pragma unroll
            for(int j = 0; j < TN; ++j)
            {
#pragma unroll
                for(int v = 0; v < 16; ++v)
                {
                    acc[i][j][v] = 0.0f;
                }
            }
        }

        stage_a sa;
        stage_b sb;

        const int row_in_wave_a = wave_m * WTM + lane_lo;
        const int row_in_wave_b = wave_n * WTN + lane_lo;

        if(step_begin < step_end)
        {
            int k0 = step_begin * BK;
            sa.fetch(a_tile + k0 * a_sk, a_sr, a_sk, rows_a, args.K - k0, tid);
            sb.fetch(b_tile + k0 * b_sk, b_sr, b_sk, rows_b, args.K - k0, tid);
            sa.commit(lds, tid);
            sb.commit(lds + A_TILE, tid);
            __syncthreads();

            int cur = 0;
            for(int step = step_begin; step < step_end; ++step)
            {
                const bool more = step + 1 < step_end;
                if(more)
                {
                    k0 = (step + 1) * BK;
                    sa.fetch(a_tile + k0 * a_sk, a_sr, a_sk, rows_a, args.K - k0, tid);
                    sb.fetch(b_tile + k0 * b_sk, b_sr, b_sk, rows_b, args.K - k0, tid);
                }
                const u32x4* lds_a = lds + cur * STAGE;
                compute_stage(lds_a, lds_a + A_TILE, acc, row_in_wave_a, row_in_wave_b, lane_hi);
                if(more)
                {
                    u32x4* nxt = lds + (cur ^ 1) * STAGE;
                    sa.commit(nxt, tid);
                    sb.commit(nxt + A_TILE, tid);
                }
                __syncthreads();
                cur ^= 1;
            }
        }

        // Epilogue.  Accumulator register v of a 32x32 tile holds row
        // 8*(v/4) + 4*(lane/32) + v%4 and column lane%32.
        const bool guarded = MODE != load_mode::vec_unguarded;
        if(w.slices == 1)
        {
            OutT* C = static_cast<OutT*>(args.C) + batch * args.batch_stride_c;
#pragma unroll
            for(int i = 0; i < TM; ++i)
            {
#pragma unroll
                for(int j = 0; j < TN; ++j)
                {
                    const int col = col0 + wave_n * WTN + j * 32 + lane_lo;
#pragma unroll
                    for(int v = 0; v < 16; ++v)
                    {
                        const int row
                            = row0 + wave_m * WTM + i * 32 + 8 * (v / 4) + 4 * lane_hi + (v % 4);
                        if(!guarded || (row < args.M && col < args.N))
                        {
                            C[(long long)row * args.N + col] = to_out<OutT>(acc[i][j][v]);
                        }
                    }
                }
            }
        }
        else
        {
            // split-K: fp32 partial sums, reduced by a second kernel.
            long long pitch;
            float*    P = partial_base<BM, BN>(args, w, batch, row0, col0, pitch);
#pragma unroll
            for(int i = 0; i < TM; ++i)
            {
#pragma unroll
                for(int j = 0; j < TN; ++j)
                {
                    const int col = col0 + wave_n * WTN + j * 32 + lane_lo;
#pragma unroll
                    for(int v = 0; v < 16; ++v)
                    {
                        const int row
                            = row0 + wave_m * WTM + i * 32 + 8 * (v / 4) + 4 * lane_hi + (v % 4);
                        if(!guarded || (row < args.M && col < args.N))
                        {
                            P[(long long)row * pitch + col] = acc[i][j][v];
                        }
                    }
                }
            }
        }
    }
};

template<class Impl>
__global__ void __launch_bounds__(Impl::THREADS) gemm_entry(const gemm_args args)
{
    Impl::run(args);
}

// Sums the k_slices fp32 partial planes of split-K in ascending slice order and
// writes C (row-major M x N per batch entry) in its own element type.
template<class OutT>
__global__ void __launch_bounds__(256) reduce_partials(OutT* __restrict__ C,
                                                       const float* __restrict__ partials,
                                                       long long plane, // M*N
                                                       int       k_slices,
                                                       long long batch_stride_c)
{
    const long long batch = blockIdx.y;
    const float*    P     = partials + batch * k_slices * plane;
    OutT*           out   = C + batch * batch_stride_c;
    for(long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < plane;
        i += (long long)gridDim.x * blockDim.x)
    {
        float s = 0.0f;
        for(int k = 0; k < k_slices; ++k)
        {
            s += P[k * plane + i];
        }
        out[i] = to_out<OutT>(s);
    }
}

// The same for the compact layout of a split tail (gemm_args::tail_begin > 0): a
// workgroup sums k_slices partial values for 4096 consecutive elements of one split
// tile (blockIdx.x = tile * chunks + chunk) and writes those that lie inside C.  Few
// tiles are split, so the work is cut fine enough to spread over the CUs and each
// thread keeps 4 independent 16-byte loads per slice in flight.
constexpr int reduce_chunk_elems = 4096;

template<class OutT>
__global__ void __launch_bounds__(256) reduce_split_tiles(OutT* __restrict__ C,
                                                          const float* __restrict__ partials,
                                                          int       M,
                                                          int       N,
                                                          int       block_m,
                                                          int       block_n,
                                                          int       grid_m,
                                                          int       grid_n,
                                                          int       group,
                                                          int       tail_begin,
                                                          int       k_slices,
                                                          long long batch_stride_c)
{
    const long long  batch       = blockIdx.y;
    const long long  split_tiles = grid_m * grid_n - tail_begin;
    const int        elems       = block_m * block_n;
    const int        chunks      = elems / reduce_chunk_elems;
    const int        tile        = blockIdx.x / chunks;
    const int        chunk       = blockIdx.x - tile * chunks;
    const tile_coord t           = map_tile(tail_begin + tile, grid_m, grid_n, group);
    const int        row0 = t.m * block_m, col0 = t.n * block_n;
    const float*     P   = partials + (batch * split_tiles + tile) * k_slices * (long long)elems;
    OutT*            out = C + batch * batch_stride_c;
    f32x4            s[4];
#pragma unroll
    for(int u = 0; u < 4; ++u)
    {
        s[u] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    const int e0 = chunk * reduce_chunk_elems + threadIdx.x * 4;
    for(int k = 0; k < k_slices; ++k)
    {
#pragma unroll
        for(int u = 0; u < 4; ++u)
        {
            s[u] += *reinterpret_cast<const f32x4*>(P + (long long)k * elems + e0 + u * 1024);
        }
    }
#pragma unroll
    for(int u = 0; u < 4; ++u)
    {
        const int e   = e0 + u * 1024;
        const int row = row0 + e / block_n, col = col0 + e % block_n; // block_n % 4 == 0
#pragma unroll
        for(int v = 0; v < 4; ++v)
        {
            if(row < M && col + v < N)
            {
                out[(long long)row * N + col + v] = to_out<OutT>(s[u][v]);
            }
        }
    }
}

// Adds up the parts of the tiles that a persistent kernel walking by K tile
// (gemm_args::stream_units > 0) left in the workgroups' fp32 slots.  Workgroup w worked
// on K tiles [w * units, (w + 1) * units) of the sequence in which tile number t (walk
// order, batch entries one after the other) holds K tiles [t * k_tiles, (t + 1) * k_tiles).
// A tile inside one range went to C whole and is skipped here; of any other tile,
// workgroup w's part is in slot 2w if the part holds the first K tile of w's range,
// else in slot 2w + 1.  Parts are added in ascending order of w.  blockIdx.x = tile *
// chunks + chunk, 4096 elements per chunk as in reduce_split_tiles.
template<class OutT>
__global__ void __launch_bounds__(256) reduce_stream_tiles(OutT* __restrict__ C,
                                                           const float* __restrict__ partials,
                                                           int       M,
                                                           int       N,
                                                           int       block_m,
                                                           int       block_n,
                                                           int       grid_m,
                                                           int       grid_n,
                                                           int       group,
                                                           int       k_tiles,
                                                           int       units,
                                                           long long batch_stride_c)
{
    const int elems    = block_m * block_n;
    const int chunks   = elems / reduce_chunk_elems;
    const int tile_lin = blockIdx.x / chunks;
    const int chunk    = blockIdx.x - tile_lin * chunks;
    const int k_first  = tile_lin * k_tiles;
    const int first    = k_first / units;
    const int last     = (k_first + k_tiles - 1) / units;
    if(first == last)
    {
        return;
    }
    const int        tiles = grid_m * grid_n;
    const int        batch = tile_lin / tiles;
    const tile_coord t     = map_tile(tile_lin - batch * tiles, grid_m, grid_n, group);
    const int        row0 = t.m * block_m, col0 = t.n * block_n;
    OutT*            out = C + batch * batch_stride_c;
    f32x4            s[4];
#pragma unroll
    for(int u = 0; u < 4; ++u)
    {
        s[u] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    const int e0 = chunk * reduce_chunk_elems + threadIdx.x * 4;
    for(int w = first; w <= last; ++w)
    {
        const long long slot = 2 * (long long)w + (w * units >= k_first ? 0 : 1);
        const float*    P    = partials + slot * elems;
#pragma unroll
        for(int u = 0; u < 4; ++u)
        {
            s[u] += *reinterpret_cast<const f32x4*>(P + e0 + u * 1024);
        }
    }
    typedef OutT out4 __attribute__((ext_vector_type(4)));
    const bool vector_ok = (N & 3) == 0 && ((unsigned long long)out & (sizeof(out4) - 1)) == 0;
#pragma unroll
    for(int u = 0; u < 4; ++u)
    {
        const int e   = e0 + u * 1024;
        const int row = row0 + e / block_n, col = col0 + e % block_n; // block_n % 4 == 0
        if(vector_ok && row < M && col + 3 < N)
        {
            out4 o;
#pragma unroll
            for(int v = 0; v < 4; ++v)
            {
                o[v] = to_out<OutT>(s[u][v]);
            }
            *reinterpret_cast<out4*>(out + (long long)row * N + col) = o;
        }
        else
        {
#pragma unroll
            for(int v = 0; v < 4; ++v)
            {
                if(row < M && col + v < N)
                {
                    out[(long long)row * N + col + v] = to_out<OutT>(s[u][v]);
                }
            }
        }
    }
}

// Copies a dense 2-D array of 16-bit elements (`outer` rows of `inner` contiguous
// elements, any alignment down to 2 bytes) into a zero-padded one whose rows are
// `inner_pad` long (a multiple of 8) and 16-byte aligned and which has `outer_pad` rows.
// Lets ragged or misaligned operands take the direct-to-LDS kernels, which need whole
// tiles and aligned rows; the zero padding along K adds nothing to the products.
// A thread writes one 16-byte piece.  It reads the two aligned 16-byte blocks that hold
// the piece's 8 source elements (the second only if it starts before the end of the
// source row) and shifts them into place; an aligned block that holds an element of the
// array lies in that element's page, so nothing is read from a page the array is not on.
// One array to copy: see pack_padded.
struct pack_job
{
    const void* src;
    void*       dst;
    int         outer, inner; // source rows and row length
    int         outer_pad, inner_pad; // the same of the copy
    long long   src_batch_stride, dst_batch_stride; // elements
};

// blockIdx.y picks the job (both operands of a GEMM go in one launch), blockIdx.z the
// batch entry.
template<class Elem16>
__global__ void __launch_bounds__(256) pack_padded(const pack_job first_job, const pack_job second_job)
{
    static_assert(sizeof(Elem16) == 2, "16-bit elements only");
    const pack_job& job       = blockIdx.y == 0 ? first_job : second_job;
    const int       outer     = job.outer;
    const int       inner     = job.inner;
    const int       outer_pad = job.outer_pad;
    const int       inner_pad = job.inner_pad;
    const Elem16*   s = static_cast<const Elem16*>(job.src) + blockIdx.z * job.src_batch_stride;
    u32x4*          d = reinterpret_cast<u32x4*>(static_cast<Elem16*>(job.dst) + blockIdx.z * job.dst_batch_stride);
    const int     pieces = inner_pad / 8;
    // (all pieces of the copy in one sequence, so that small arrays still fill workgroups)
    const long long total = (long long)outer_pad * pieces;
    for(long long at = (long long)blockIdx.x * blockDim.x + threadIdx.x; at < total;
        at += (long long)gridDim.x * blockDim.x)
    {
        {
            const int o = static_cast<int>(at / pieces);
            const int i = static_cast<int>(at - (long long)o * pieces);
            u32x4 out = {0u, 0u, 0u, 0u};
            if(o < outer && 8 * i < inner)
            {
                const unsigned long long first = reinterpret_cast<unsigned long long>(s + (long long)o * inner + 8 * i);
                const unsigned long long end   = reinterpret_cast<unsigned long long>(s + (long long)(o + 1) * inner);
                const u32x4*             block = reinterpret_cast<const u32x4*>(first & ~15ull);
                const u32x4              b0    = block[0];
                u32x4                    b1    = {0u, 0u, 0u, 0u};
                if((first & 15ull) != 0 && reinterpret_cast<unsigned long long>(block + 1) < end)
                {
                    b1 = block[1];
                }
                const unsigned int w[8] = {b0[0], b0[1], b0[2], b0[3], b1[0], b1[1], b1[2], b1[3]};
                const int          q    = static_cast<int>(first & 15ull) >> 2; // whole words to skip
                const bool         half = (first & 2ull) != 0; // and half a word more
                const int          valid = inner - 8 * i; // elements of the piece that the row holds
#pragma unroll
                for(int k = 0; k < 4; ++k)
                {
                    unsigned int lo = w[k], hi = w[k + 1];
#pragma unroll
                    for(int t = 1; t < 4; ++t)
                    {
                        lo = q == t ? w[k + t] : lo;
                        hi = q == t ? w[k + t + 1] : hi;
                    }
                    unsigned int v = half ? (lo >> 16) | (hi << 16) : lo;
                    if(2 * k + 1 >= valid)
                    {
                        v &= 2 * k >= valid ? 0u : 0xffffu;
                    }
                    out[k] = v;
                }
            }
            d[(long long)o * pieces + i] = out;
        }
    }
}

template<class OutT>
__global__ void __launch_bounds__(256) fill_zero(OutT* __restrict__ C, long long count)
{
    for(long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < count;
        i += (long long)gridDim.x * blockDim.x)
    {
        C[i] = to_out<OutT>(0.0f);
    }
}

} // namespace device
} // namespace rocm_wmma_gemm

#endif // ROCM_WMMA_GEMM_GEMM_KERNEL_HPP
