// Shape -> launch plan.  The tuned table comes from gemm_config_gfx950_*.json via
// config/generate_config.py; shapes the table does not name are served by a time
// estimate over the compiled variants when they are regular (select_plan: K a multiple
// of 64, extents multiples of 8), else by the table's nearest entry, and layouts the
// table does not cover at all by a shape heuristic.
//
// select_plan_from follows the reference's generated find_best_config /
// find_closest_config (reference rocm_wmma_gemm/config/generate_config.py:174-271):
//   1. exact (M, N, K, type group, layouts) hit;
//   2. for the fp32-output group, an exact hit in the 16-bit-output group;
//   3. nearest entry with the same type group and layouts: nearest K first, then
//      smallest squared (M, N) distance; an empty group falls back to group 0.
// Unlike the reference there is no sentinel index doubling as "not found", so a
// genuine hit on any entry is honoured.
#ifndef ROCM_WMMA_GEMM_CONFIG_SELECT_HPP
#define ROCM_WMMA_GEMM_CONFIG_SELECT_HPP

#include <cstddef>

namespace rocm_wmma_gemm
{
namespace host
{

struct launch_plan
{
    int variant; // index into the compiled variant table
    int swizzle; // band height of the tile map: s > 0 bands of s tile rows, s < 0 bands of -s tile columns
    int split_k; // K slices (1 = off); -s (s > 1) = split only the last, partial wave of tiles s
                 // ways; -1 = persistent kernel walks by K tile (equal K tiles per workgroup)
    int touch = 0; // persistent kernel, two small fields.  Bits 0-3: d > 0 = touch the cache lines of
                   // the K tile d tiles past the one being loaded (see gemm_args::warm_ahead); 0 = off.
                   // Bits 4-7: c > 0 = walk the K tiles in runs of 2^(c-1), the XCDs out of step by
                   // whole runs (see gemm_args::k_block); 0 = in order.
                   // Bits 8-9: c > 0 = within groups of 2^c K tiles the workgroups start at different
                   // tiles (see gemm_args::k_group); 0 = in order.
};

// the two fields of launch_plan::touch
constexpr int plan_touch_distance(int touch)
{
    return touch & 15;
}
constexpr int plan_k_run(int touch)
{
    return ((touch >> 4) & 15) == 0 ? 0 : 1 << (((touch >> 4) & 15) - 1);
}
constexpr int plan_k_group(int touch)
{
    return ((touch >> 8) & 3) == 0 ? 0 : 1 << ((touch >> 8) & 3);
}
// run: 0 or a power of two up to 16; group: 0, 2, 4 or 8
constexpr int plan_touch_field(int distance, int run, int group = 0)
{
    int code = 0;
    for(int r = run; r > 0; r >>= 1)
    {
        ++code;
    }
    return (distance & 15) | (code << 4) | ((group == 2 ? 1 : group == 4 ? 2 : group == 8 ? 3 : 0) << 8);
}

struct tuned_entry
{
    size_t m, n, k;
    int    type_group; // 0: C is 16-bit (f16_f16, bf16_bf16); 1: C is fp32
    int    layout_a, layout_b, layout_c; // 0 row-major, 1 column-major
    launch_plan plan;
};

// Constants of model_plan's time estimate (microseconds, bytes per microsecond), measured
// on the GPU: config/fit_model.py fits them to a tuner log, config/model_<arch>.json keeps
// them and config/generate_config.py copies them into the generated header.
struct model_step
{
    int    pipeline, block_m, block_n;
    double step_us; // per K tile of 64 with every compute unit at work
    double item_us; // per tile: the stores of C and the turn to the next tile
};
// Constants of the estimate for the plans of the whole-K streaming kernel (pipeline 7),
// fitted by config/fit_model.py --stream to a sweep of config/sweep_stream.py.
struct model_stream
{
    double launch_us, fill_us; // per launch; per pass over the compute units (the ring fills)
    double exchange_us; // several workgroups per tile: the partial tiles through memory ...
    double exchange_us_per_kb; // ... and per KiB of them that the last workgroup adds up
    double bytes_per_us_kmajor, bytes_per_us_other; // stream of the large operand from memory
    double bytes_per_us_l2; // the small operand, which every workgroup reads from L2
    double transposed_operand; // relative cost of a stage per operand that is not K-contiguous
    double panel_sharing; // how much of a panel of the large operand that g workgroups read
                          // is fetched once for all: it counts as fetched g / (1 + (g - 1) x this) times
    double half_line; // factor on a rate for an operand contiguous along M or N on a 32-wide side
                      // of the tile: requests of 64 bytes, half a cache line
    double beyond_cache, beyond_cache_other; // factors on the two rates from memory for a large
                         // operand over 256 MB, K-contiguous or not (set by hand, not fitted)
    double taking_turns; // two workgroups on a compute unit: a stage of each takes 1 + this of what
                         // it takes alone, where the compute unit is the bound (set by hand)
    double stage_us[8]; // per stage of 128 of one compute unit: tiles 32x32, 64x32, 32x64, 64x64,
                        // 16x32, 16x64, 32x16, 64x16
};
struct model_constants
{
    int    compute_units; // of the GPU the constants were measured on
    double launch_us, reduce_us;
    double plane_bytes_per_us; // split-K partial planes: written, then read by the reduce kernel
    double tile_bytes_per_us; // partial tiles of a split tail wave or of the walk by K tile
    double copy_bytes_per_us; // padded operand copies
    double operand_bytes_per_us; // what the tiled kernels reach at most streaming A and B from memory
                                 // (skinny shapes: 134 MB in 24-27 us of split-K kernel, 470 MB in 83-96; set by hand)
    const model_step* steps;
    int               step_count;
    model_stream      stream;
};
extern const model_constants model_measured;

// Defined in config_select.cpp
extern const tuned_entry* const tuned_table;
extern const size_t             tuned_count;

// Pure functions over a table (unit-testable with any table).
bool find_exact(const tuned_entry* table, size_t count, size_t m, size_t n, size_t k,
                int type_group, int la, int lb, int lc, launch_plan* out);
bool find_closest(const tuned_entry* table, size_t count, size_t m, size_t n, size_t k,
                  int type_group, int la, int lb, int lc, launch_plan* out);
launch_plan heuristic_plan(size_t m, size_t n, size_t k, int lc);
// Estimated-time choice among the compiled variants for a shape without a tuned entry;
// false for shapes it does not cover (ragged K, odd extents).
// cus: compute units of the GPU the plan is for (0: the GPU the constants were measured on).
bool model_plan(size_t m, size_t n, size_t k, int lc, int la, int lb, launch_plan* out, size_t batch = 1,
                size_t cus = 0);
// The streaming kernel's plans alone (skinny shapes: one extent at most 128, or small ones:
// at most 2^20 elements of C; K at least 256, a multiple of 8 where an operand is
// K-contiguous), in kernel space (rows x cols, the operands' K-contiguity): the cheapest by
// estimate and its microseconds; false when no compiled variant takes the problem.
bool stream_plan(size_t rows, size_t cols, size_t k, bool a_kmajor, bool b_kmajor, size_t batch, size_t cus,
                 launch_plan* out, double* microseconds);
launch_plan select_plan_from(const tuned_entry* table, size_t count, size_t m, size_t n, size_t k,
                             int type_idx, int lc, int la, int lb);

inline int type_group_of(int type_idx)
{
    return (type_idx == 1 || type_idx == 3) ? 1 : 0;
}

launch_plan select_plan(size_t m, size_t n, size_t k, int type_idx, int lc, int la, int lb, size_t batch = 1,
                        size_t cus = 0);

} // namespace host
} // namespace rocm_wmma_gemm

#endif
