/*
 * C ABI of librocm_wmma_gemm_gfx950.so -- the drop-in boundary of the GEMM path.
 *
 * The first four functions are exactly the symbols the reference's runtime
 * loader resolves with dlsym (reference rocm_wmma_gemm/include/rocm_wmma_gemm/
 * kernel_loader.hpp:53-54,110-113) and that its arch library defines
 * (reference rocm_wmma_gemm/src/gemm.cpp:219-250).  The rest are additions with
 * no counterpart in the reference: introspection and tuning hooks.
 *
 * Conventions for every gemm entry point:
 *   C (M x N) = A (M x K) * B (K x N); C is overwritten; operands are dense and
 *   packed in the stated layout; layout_* is 0 for row-major, 1 for column-major;
 *   batch b uses A + b*M*K, B + b*K*N, C + b*M*N (elements);
 *   `stream` is the ADDRESS of the caller's hipStream_t (a hipStream_t*), not the
 *   handle itself; the work is enqueued there and the call returns at once;
 *   all pointers are device pointers owned by the caller;
 *   a layout value outside {0,1} makes the call a no-op (reference behaviour,
 *   src/gemm.cpp:243); M, N or batch_count of 0 is a no-op; K of 0 zero-fills C.
 */
#ifndef ROCM_WMMA_GEMM_C_H
#define ROCM_WMMA_GEMM_C_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* fp16 A,B -> fp16 C.  Replaces reference src/gemm.cpp:247 (DEFINE_C_DISPATCH(f16_f16, half, half)). */
void rocm_wmma_gemm_f16_f16(void* C, void* A, void* B, size_t M, size_t N, size_t K,
                            size_t batch_count, int layout_c, int layout_a, int layout_b,
                            void* stream);

/* fp16 A,B -> fp32 C.  Replaces reference src/gemm.cpp:248. */
void rocm_wmma_gemm_f32_f16(void* C, void* A, void* B, size_t M, size_t N, size_t K,
                            size_t batch_count, int layout_c, int layout_a, int layout_b,
                            void* stream);

/* bf16 A,B -> bf16 C.  Replaces reference src/gemm.cpp:249. */
void rocm_wmma_gemm_bf16_bf16(void* C, void* A, void* B, size_t M, size_t N, size_t K,
                              size_t batch_count, int layout_c, int layout_a, int layout_b,
                              void* stream);

/* bf16 A,B -> fp32 C.  Replaces reference src/gemm.cpp:250. */
void rocm_wmma_gemm_f32_bf16(void* C, void* A, void* B, size_t M, size_t N, size_t K,
                             size_t batch_count, int layout_c, int layout_a, int layout_b,
                             void* stream);

/* ---- additions (no counterpart in the reference) ------------------------ */

/* type_idx values, in the reference launcher's order (kernel_launcher.hpp:78-83). */
#define ROCM_WMMA_GEMM_TYPE_F16_F16 0
#define ROCM_WMMA_GEMM_TYPE_F32_F16 1
#define ROCM_WMMA_GEMM_TYPE_BF16_BF16 2
#define ROCM_WMMA_GEMM_TYPE_F32_BF16 3

/* Status codes of the additions that return int (the four reference entry points return
 * void, as in the reference). */
#define ROCM_WMMA_GEMM_OK 0
#define ROCM_WMMA_GEMM_ERR_VARIANT (-1)  /* the forced variant cannot run this problem */
#define ROCM_WMMA_GEMM_ERR_ARGUMENT (-2) /* type index, variant index or layout code out of range */
#define ROCM_WMMA_GEMM_ERR_SCRATCH (-3)  /* the call needs more scratch memory than the fixed buffer holds */
#define ROCM_WMMA_GEMM_ERR_RUNTIME (-4)  /* the HIP runtime reported an error (symbol lookup, launch) */
#define ROCM_WMMA_GEMM_ERR_LIMIT (-5)    /* M, N or K beyond 31 bits, tile grid too large, or no kernel built */

/* Description of one compiled kernel variant. */
typedef struct rocm_wmma_gemm_variant_info
{
    int block_m, block_n, block_k; /* workgroup tile */
    int warps_m, warps_n;          /* wave grid inside the workgroup */
    int warp_tile_m, warp_tile_n;  /* 32x32 MFMA tiles per wave (0: a 16-wide side of the streaming kernel's tile) */
    int pipeline;                  /* 0 = register-staged general path, 1 = direct-to-LDS, 2 = direct-to-LDS ping-pong, 3, 4 = 1, 2 on the 16x16x32 MFMA, 5 = one wave per SIMD, persistent workgroups, 6 = 1 with a ring of 4 tiles at BLOCK_K 64, 7 = whole-K streaming kernel (tiles of 16 to 128 rows by 16 to 64 columns, one workgroup per tile over all of K, for skinny and small problems) */
    int lds_bytes;                 /* static LDS per workgroup */
    int threads;                   /* workgroup size */
} rocm_wmma_gemm_variant_info;

/* "gfx950": the architecture this library was compiled for. */
const char* rocm_wmma_gemm_arch(void);

/* Number of compiled tile variants; fills *info for variant in [0, count). Returns 0 on success. */
int rocm_wmma_gemm_variant_count(void);
int rocm_wmma_gemm_variant_info_get(int variant, rocm_wmma_gemm_variant_info* info);

/* Which variant the dispatcher would pick for this problem (the table built from
 * gemm_config_gfx950_*.json, then shape heuristics).  type_idx as above.
 * Also reports the swizzle (band height of the tile walk: g > 0 bands of g tile rows,
 * g < 0 bands of -g tile columns) and the split field: s > 1 = every
 * tile's K range is cut into s slices (added up by a second kernel; on the whole-K streaming
 * kernel, pipeline 7, s = 2, 4 or 8 workgroups share a tile and the last of them to finish
 * adds the parts up inside the one launch); -s < -1 = only the tiles of the last, partial
 * wave over the compute units are cut into s slices; -1 = the persistent kernel's
 * workgroups each take the same number of K tiles of the sequence of all K tiles of the
 * launch, wherever the tile borders fall, and the cut tiles are added up afterwards (other
 * kernels read -1 as 1); 1 = no split.  Returns the variant index, or -1 for invalid
 * arguments. */
int rocm_wmma_gemm_select(size_t M, size_t N, size_t K, int type_idx, int layout_c, int layout_a,
                          int layout_b, int* swizzle, int* split_k);
/* The same for a strided batch of batch_count problems of this shape: the dispatcher counts
 * the tiles of the whole batch when it weighs tile sizes and splits, so the answer can differ
 * from the single problem's. */
int rocm_wmma_gemm_select_batched(size_t M, size_t N, size_t K, size_t batch_count, int type_idx,
                                  int layout_c, int layout_a, int layout_b, int* swizzle,
                                  int* split_k);

/* rocm_wmma_gemm_select_batched, also reporting the plan's fourth field: touch_ahead d > 0 =
 * the persistent kernel, beside the loads of a K tile, touches the cache lines of the K tile
 * d tiles further on (one dword per line from two waves of each workgroup, the workgroups
 * that share an operand panel touching different quarters), so that those lines are on
 * their way into the XCD's L2 a tile time before the loads that need them; it pays for a
 * long K whose operands outgrow the memory-side cache and costs a few percent elsewhere,
 * so the tuner decides.  0 = off; other kernels ignore it.  The value carries a second small
 * field in bits 4-7: c > 0 = the persistent kernel walks the K tiles of a tile in runs of
 * 2^(c-1) and, within every 8 runs, the workgroups of XCD x start at run x and wrap round,
 * so that the XCDs that share an operand panel are never on the same run (each finds in the
 * memory-side cache what another fetched first, instead of all of them waiting for memory at
 * once); the sums of an element are added in that order, the same in every call.  Worth
 * 7-10 % on operands beyond that cache with a K-contiguous operand, nothing elsewhere.  And a
 * third in bits 8-9: c > 0 = within every aligned group of 2^c K tiles the workgroup of tile
 * (i, j) starts at tile (i + j) mod 2^c of the group and wraps round, so that the workgroups
 * of an XCD that share an operand panel ask for a line at different times and all but the
 * first find it in L2: worth 14-17 % on the same problems; the dispatcher's estimate sets
 * groups of 4 there, the tuner decides per entry.  Both leave the sums of an element in one
 * fixed order, the same in every call.  (JSON keys: "touch_ahead" for bits 0-3, "k_runs" for
 * the run length, "k_group" for the group size.) */
int rocm_wmma_gemm_select_ex(size_t M, size_t N, size_t K, size_t batch_count, int type_idx, int layout_c,
                             int layout_a, int layout_b, int* swizzle, int* split_k, int* touch_ahead);

/* Same computation as the four entry points above, but with the tile variant,
 * swizzle and split field (see above) forced (tuner hook).  Returns ROCM_WMMA_GEMM_OK,
 * ROCM_WMMA_GEMM_ERR_VARIANT if the variant cannot run this problem, or another of the
 * status codes above. */
int rocm_wmma_gemm_run_variant(int type_idx, int variant, int swizzle, int split_k, void* C,
                               void* A, void* B, size_t M, size_t N, size_t K,
                               size_t batch_count, int layout_c, int layout_a, int layout_b,
                               void* stream);

/* rocm_wmma_gemm_run_variant with the plan's touch_ahead field (both parts of it) forced too
 * (see rocm_wmma_gemm_select_ex). */
int rocm_wmma_gemm_run_variant_ex(int type_idx, int variant, int swizzle, int split_k, int touch_ahead,
                                  void* C, void* A, void* B, size_t M, size_t N, size_t K,
                                  size_t batch_count, int layout_c, int layout_a, int layout_b,
                                  void* stream);

/* Adds a tile variant that was compiled outside this library (the tuner builds
 * rocm_wmma_gemm_amd/csrc/kernel_jit.hip for one tuple, type pair and pair of operand layouts
 * and passes that library's rwg_jit_kernels here: nine entry points, for the three load modes,
 * 16-byte unguarded, 16-byte guarded, 2-byte, then the twins of the first two that walk K in
 * runs (see rocm_wmma_gemm_select_ex), then those twins with non-temporal loads of B and of A;
 * null where the pipeline or tile has none).  The
 * variant gets the next index after the compiled ones and runs through
 * rocm_wmma_gemm_run_variant like any other; registering the same tuple again for another
 * type pair or layout pair adds those kernels to the same index.  operand *_kmajor: 1 if K is
 * the operand's contiguous dimension in the kernel's view (C row-major: A row-major, B
 * column-major; a column-major C swaps the operands).  Returns the variant index,
 * ROCM_WMMA_GEMM_ERR_VARIANT if the library already holds a compiled variant of this
 * description, ROCM_WMMA_GEMM_ERR_ARGUMENT for a tuple no kernel can have, or
 * ROCM_WMMA_GEMM_ERR_LIMIT when 64 variants have been registered.  The library that holds
 * the kernels must stay loaded.  The role of the reference tuner's run-time compilation
 * (reference rocm_wmma_gemm/config/tuner.cpp:237-454), split into compile (tuner) and
 * launch (library). */
int rocm_wmma_gemm_register_variant(int block_m, int block_n, int block_k, int warps_m, int warps_n,
                                    int pipeline, int type_idx, int a_kmajor, int b_kmajor,
                                    const void* const* kernels);

/* Gives the current device's library-owned scratch buffer back (split-K partial sums and
 * padded operand copies live there: 256 MiB from the first call that needs it, more when a
 * call needs more).  Waits for the device to finish first.  Returns 0 when the buffer is
 * gone or was never there, 1 when it was kept because a call on a capturing stream has
 * used it (a graph may hold its address), ROCM_WMMA_GEMM_ERR_RUNTIME without a device.
 * The next call that needs scratch memory allocates again.  Also puts the arrival counters
 * of shared tiles back to zero (they return to zero by themselves after every launch that
 * runs to its end; a kernel killed in flight may leave one counting, which later launches
 * ignore anyway because every launch tags its counts).  No counterpart in the reference,
 * which owns no memory. */
int rocm_wmma_gemm_workspace_release(void);

/* Size of the fixed per-GPU scratch buffer behind rocm_wmma_gemm_noalloc. */
#define ROCM_WMMA_GEMM_NOALLOC_SCRATCH_BYTES (64u << 20)

/* The same computation as the four reference entry points (type_idx picks the type pair),
 * for callers that cannot allocate device memory: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference, whose
 * kernels need no scratch memory at all.  Here split-K partial sums and zero-padded copies
 * of ragged operands do; the other entry points keep them in a buffer that the library
 * allocates and grows on demand, this one keeps them in a fixed array of
 * ROCM_WMMA_GEMM_NOALLOC_SCRATCH_BYTES that is part of the library's code object on every
 * GPU (held from the first use of the library on that GPU until the process ends), and
 * calls neither hipMalloc nor hipFree nor anything else that allocates.
 *   - A call whose plan needs more scratch memory than the array holds fails with
 *     ROCM_WMMA_GEMM_ERR_SCRATCH and enqueues nothing (of the shapes the library is
 *     tuned for: K = 65536 at M = N = 1024, which wants 128 MiB of partial tiles, and
 *     (4095, 5121, 3001), which wants 56 MiB of padded copies plus its partial tiles).
 *     Calls that need no scratch memory (whole tiles, no split) have no size limit.
 *   - The first call on a GPU looks the array's address up (hipGetSymbolAddress); make that
 *     call outside graph capture.
 *   - Every call on a GPU uses that GPU's one array, which keeps the previous call's
 *     contents; nothing has to start at zero (each kernel writes what a later one reads).
 *     Calls of THIS entry point that overlap on one GPU (two streams, two threads, replays
 *     of two captured graphs) race on the array and on the arrival counters of shared
 *     tiles that go with it: order them.  Calls of the other entry points may overlap with
 *     them freely: those use the library's allocated buffer and counters of their own.
 * Returns ROCM_WMMA_GEMM_OK or one of the codes above; a layout code outside {0, 1} is
 * ROCM_WMMA_GEMM_ERR_ARGUMENT here rather than a silent no-op. */
int rocm_wmma_gemm_noalloc(int type_idx, void* C, void* A, void* B, size_t M, size_t N, size_t K,
                           size_t batch_count, int layout_c, int layout_a, int layout_b,
                           void* stream);

#ifdef __cplusplus
}
#endif

#endif /* ROCM_WMMA_GEMM_C_H */
