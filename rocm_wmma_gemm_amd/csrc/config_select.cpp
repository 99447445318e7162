// Implementation of the shape -> launch plan lookup (plain C++, no device code).
#include "config_select.hpp"

#include <algorithm>

#include <initializer_list>
#include <limits>

#include "config_generated.hpp"

namespace rocm_wmma_gemm
{
namespace host
{

const tuned_entry* const tuned_table = generated::entries;
const size_t             tuned_count = generated::entry_count;
const model_constants    model_measured
    = {generated::model_compute_units,      generated::model_launch_us,
       generated::model_reduce_us,          generated::model_plane_bytes_per_us,
       generated::model_tile_bytes_per_us,  generated::model_copy_bytes_per_us,
       generated::model_operand_bytes_per_us,
       generated::model_steps,              generated::model_step_count,
       generated::model_stream_constants};

namespace
{
bool same_slot(const tuned_entry& e, int type_group, int la, int lb, int lc)
{
    return e.type_group == type_group && e.layout_a == la && e.layout_b == lb && e.layout_c == lc;
}
} // namespace

bool find_exact(const tuned_entry* table, size_t count, size_t m, size_t n, size_t k,
                int type_group, int la, int lb, int lc, launch_plan* out)
{
    for(size_t i = 0; i < count; ++i)
    {
        const tuned_entry& e = table[i];
        if(e.m == m && e.n == n && e.k == k && same_slot(e, type_group, la, lb, lc))
        {
            *out = e.plan;
            return true;
        }
    }
    return false;
}

bool find_closest(const tuned_entry* table, size_t count, size_t m, size_t n, size_t k,
                  int type_group, int la, int lb, int lc, launch_plan* out)
{
    bool   any       = false;
    size_t best_kgap = std::numeric_limits<size_t>::max();
    size_t best_k    = 0;
    for(size_t i = 0; i < count; ++i)
    {
        const tuned_entry& e = table[i];
        if(!same_slot(e, type_group, la, lb, lc))
        {
            continue;
        }
        any              = true;
        const size_t gap = e.k > k ? e.k - k : k - e.k;
        if(gap < best_kgap)
        {
            best_kgap = gap;
            best_k    = e.k;
        }
    }
    if(!any)
    {
        return false;
    }
    double best_d = std::numeric_limits<double>::max();
    for(size_t i = 0; i < count; ++i)
    {
        const tuned_entry& e = table[i];
        if(!same_slot(e, type_group, la, lb, lc) || e.k != best_k)
        {
            continue;
        }
        const double dm = static_cast<double>(m) - static_cast<double>(e.m);
        const double dn = static_cast<double>(n) - static_cast<double>(e.n);
        const double d  = dm * dm + dn * dn;
        if(d < best_d)
        {
            best_d = d;
            *out   = e.plan;
        }
    }
    return true;
}

launch_plan heuristic_plan(size_t m, size_t n, size_t k, int lc)
{
    // kernel-space rows/columns (column-major C runs as the transposed problem)
    const size_t rows = lc == 0 ? m : n;
    const size_t cols = lc == 0 ? n : m;
    launch_plan  plan;
    const size_t big_tiles = ((rows + 255) / 256) * ((cols + 255) / 256);
    plan.variant           = (rows >= 256 && cols >= 256 && big_tiles >= 128) ? 1 : 0;
    plan.swizzle           = 4;
    plan.split_k           = 1;
    plan.touch             = 0;
    const size_t bm        = plan.variant == 1 ? 256 : 128;
    const size_t bk        = plan.variant == 1 ? 64 : 32;
    const size_t tiles     = ((rows + bm - 1) / bm) * ((cols + bm - 1) / bm);
    const size_t k_steps   = (k + bk - 1) / bk;
    if(tiles < 128 && k_steps >= 32)
    {
        // too few tiles for 256 CUs: slice K until the chip is covered about twice,
        // keeping at least 8 K steps per slice
        size_t want = (512 + tiles - 1) / tiles;
        size_t cap  = k_steps / 8;
        size_t s    = want < cap ? want : cap;
        if(s > 64)
        {
            s = 64;
        }
        plan.split_k = s < 1 ? 1 : static_cast<int>(s);
    }
    return plan;
}

namespace
{
// Compiled variants as the model sees them.
struct model_variant
{
    int block_m, block_n, block_k, waves_m, waves_n, pipeline;
};
#define RWG_VARIANT(IDX, BM, BN, BK, WM, WN, PIPE) {BM, BN, BK, WM, WN, PIPE},
const model_variant model_variants[] = {
#include "variants.def"
};
#undef RWG_VARIANT

// Microseconds per K tile of 64 with every compute unit at work, and per tile for its
// stores: measured constants (model_measured), one pair per pipeline and tile.
bool step_cost(const model_variant& v, double* step_us, double* item_us)
{
    if(v.block_k != 64)
    {
        return false;
    }
    for(int i = 0; i < model_measured.step_count; ++i)
    {
        const model_step& s = model_measured.steps[i];
        if(s.pipeline == v.pipeline && s.block_m == v.block_m && s.block_n == v.block_n)
        {
            *step_us = s.step_us;
            *item_us = s.item_us;
            return true;
        }
    }
    return false;
}

size_t ceil_div(size_t a, size_t b)
{
    return (a + b - 1) / b;
}
} // namespace

// A plan from arithmetic instead of from the nearest tuned shape: for every compiled
// variant of the two pipelines that serve regular shapes, and every way to split, the
// time is estimated as launch + waves of tiles over the CUs x (K tiles x time per K
// tile + stores) + what the split costs in partial sums, and the cheapest wins.  What
// the nearest tuned shape cannot know is how THIS shape's tile count falls on 256 CUs:
// 3584^3 next to the tuned 3072^3 inherited its 192 x 192 tiles (361 of them, two waves
// with the second less than half full) and ran at 0.7 of the 196 tiles of 256 x 256.
// On the 208 tuned entries the model can serve, its pick is on average 2.7 % slower than
// the tuner's, 25 % at worst.
bool model_plan(size_t m, size_t n, size_t k, int lc, int la, int lb, launch_plan* out, size_t batch,
                size_t cus_of_device)
{
    const size_t rows = lc == 0 ? m : n;
    const size_t cols = lc == 0 ? n : m;
    // operands in kernel space: a column-major C runs as the transposed problem
    bool a_kmajor = la == 0, b_kmajor = lb == 1;
    if(lc != 0)
    {
        const bool t = a_kmajor;
        a_kmajor     = b_kmajor;
        b_kmajor     = t;
    }
    // K need not be whole K tiles: the persistent kernel cuts a partial last tile off
    // itself, as long as the rows of a K-contiguous operand stay 16-byte aligned
    const bool k_whole = k % 64 == 0;
    // Skinny against a large operand (decode-like: a few rows against 4096 x 4096 .. 28672
    // x 8192): the plans of the whole-K streaming kernel compete with the others by their
    // estimates, and stand alone for the shapes the others would only take through copies.
    launch_plan stream_best{};
    double      stream_us   = 0.0;
    const bool  have_stream = stream_plan(rows, cols, k, a_kmajor, b_kmajor, batch, cus_of_device, &stream_best, &stream_us);
    if(k < 64 || rows % 8 != 0 || cols % 8 != 0 || rows < 16 || cols < 16
       || (!k_whole && (a_kmajor || b_kmajor) && k % 8 != 0))
    {
        // shapes every direct kernel would only take through padded copies
        if(have_stream)
        {
            *out = stream_best;
        }
        return have_stream;
    }
    // (the constants are per compute unit at work, so the estimate carries over to a GPU
    // or partition with another count; the tile walk still assumes 8 XCDs)
    const size_t cus                = cus_of_device != 0 ? cus_of_device : static_cast<size_t>(model_measured.compute_units);
    const double launch_us          = model_measured.launch_us;
    const double reduce_us          = model_measured.reduce_us;
    const double plane_bytes_per_us = model_measured.plane_bytes_per_us; // written, then read by reduce_partials
    const double tile_bytes_per_us  = model_measured.tile_bytes_per_us; // split tail, walk by K tile
    // (small planes are paid for in latency, not bandwidth: past 32 MB the rest moves at
    // twice the rate; 8192x1024x8192 cut in two moves 134 MB in ~30 us)
    auto plane_traffic_us = [&](double bytes) {
        const double knee = 32.0 * 1024 * 1024;
        return bytes <= knee ? bytes / plane_bytes_per_us
                             : knee / plane_bytes_per_us + (bytes - knee) / (2.0 * plane_bytes_per_us);
    };
    const double operand_us = static_cast<double>((rows + cols) * k * batch) * 2.0 / model_measured.operand_bytes_per_us;
    const size_t     kt            = ceil_div(k, size_t{64});
    double           best          = 0.0;
    bool             found         = false;
    const int        count         = static_cast<int>(sizeof(model_variants) / sizeof(model_variants[0]));
    for(int i = 0; i < count; ++i)
    {
        const model_variant& v = model_variants[i];
        double               step = 0.0, item = 0.0;
        if(!step_cost(v, &step, &item))
        {
            continue;
        }
        const size_t bm = v.block_m, bn = v.block_n;
        if((bm % 128 != 0 && !a_kmajor) || (bn % 128 != 0 && !b_kmajor))
        {
            continue; // not built for this layout
        }
        if((bm >= 192 && rows < 192) || (bn >= 192 && cols < 192))
        {
            continue; // a tile much larger than the problem
        }
        if(v.pipeline == 6 && (bm == 64 || bn == 64) && rows > 128 && cols > 128)
        {
            continue; // the 64-wide tiles are for skinny shapes
        }
        // (batch entries are more tiles: the persistent kernel numbers its items over the
        // whole batch, the others put the batch in grid.y)
        const size_t tm = ceil_div(rows, bm), tn = ceil_div(cols, bn), tiles = tm * tn * batch;
        const double tile_bytes = static_cast<double>(bm * bn) * 4.0;
        // only the persistent kernel takes ragged M, N or K as they are; the others run on
        // padded copies of the operands that need them (two more launches)
        double copies_us = 0.0;
        if(v.pipeline != 5 && (rows % bm != 0 || cols % bn != 0 || !k_whole))
        {
            const double k_pad = static_cast<double>(kt * 64);
            const double elems = ((rows % bm != 0 || !k_whole ? static_cast<double>(tm * bm) * k_pad : 0.0)
                                  + (cols % bn != 0 || !k_whole ? static_cast<double>(tn * bn) * k_pad : 0.0))
                                 * static_cast<double>(batch);
            copies_us = launch_us + elems * 2.0 * 2.0 / model_measured.copy_bytes_per_us;
        }
        auto consider = [&](double t, int split) {
            t += copies_us;
            if(!found || t < best)
            {
                found        = true;
                best         = t;
                out->variant = i;
                out->swizzle = 4;
                out->split_k = split;
                // operands that outgrow the 256 MB memory-side cache and are K-contiguous (both, or
                // one of them with a K of 20480 and more: 8192 x 8192 x 16384 with B row-major loses
                // 2 % to it, x 28672 gains 5 %): the workgroups of the persistent kernel start each
                // group of 8 K tiles at different tiles.  (At 268 MB, 4096 x 4096 x 16384 and
                // 8192^3, the plain walk is level or 3 % ahead; at 335 MB the groups gain 17 %.)
                out->touch = v.pipeline == 5 && (rows + cols) * k * 2 * batch >= (size_t{300} << 20)
                                     && ((a_kmajor && b_kmajor && kt >= 64) || ((a_kmajor || b_kmajor) && kt >= 320))
                                 ? plan_touch_field(0, 0, 8)
                                 : 0;
            }
        };
        // whole tiles
        consider(launch_us + static_cast<double>(ceil_div(tiles, cus)) * (kt * step + item), 1);
        // only the last, partial wave of tiles split
        for(const size_t s : {size_t{2}, size_t{3}, size_t{4}, size_t{6}, size_t{8}})
        {
            if(v.pipeline != 5)
            {
                break;
            }
            if(tiles > cus && tiles % cus != 0 && kt / s >= 4 && (tiles % cus) * s <= cus * 5 / 4)
            {
                // (the slices of the split tiles take one more pass over the CUs, or two
                // when there are more of them than CUs)
                consider(launch_us + static_cast<double>(tiles / cus) * (kt * step + item)
                             + static_cast<double>(ceil_div((tiles % cus) * s, cus)) * (ceil_div(kt, s) * step + item)
                             + reduce_us
                             + (tiles % cus) * s * tile_bytes * 2.0 / tile_bytes_per_us,
                         -static_cast<int>(s));
            }
        }
        // every tile split (few tiles, long K)
        if(tiles < cus)
        {
            for(size_t s = 2; s <= 32; s *= 2)
            {
                if(kt / s < 4)
                {
                    break;
                }
                consider(launch_us + static_cast<double>(ceil_div(tiles * s, cus)) * (ceil_div(kt, s) * step + item)
                             + reduce_us + plane_traffic_us(s * tiles * tile_bytes * 2.0),
                         static_cast<int>(s));
            }
        }
        // the persistent kernel's walk by K tile: for few tiles and a long K only (with
        // many tiles the workgroups of an XCD stop walking K in step and lose each
        // other's operand panels in L2: 7168^3 ran at 950 TFLOP/s this way, 1250 by tile)
        if(v.pipeline == 5 && tiles * 4 <= cus && tiles * kt >= 4 * cus)
        {
            const size_t groups = tiles * kt < cus ? tiles * kt : cus;
            consider(launch_us + ceil_div(tiles * kt, groups) * step + item + reduce_us
                         + groups * 1.25 * tile_bytes * 2.0 / tile_bytes_per_us,
                     -1);
        }
    }
    // The two estimates compete for skinny shapes (up to 128 rows or columns) and for small
    // problems (at most 2^20 elements of C, K up to 4096: 512 x 2048 x 2048 12.2 against 17.8
    // us, 256 x 256 x 1024 8.6 against 12.8), in every layout.  From 65 rows on only while
    // the streaming plan's workgroups all run at once: the estimates are closer to each
    // other than to the truth where they need a second pass over the compute units
    // (128 x 14336 x 4096: 34.5 us streamed, 29.2 tiled; 128 x 8192 x 8192, one pass, 30.3
    // against 37.4).
    bool one_pass = false;
    if(have_stream)
    {
        const model_variant& v      = model_variants[stream_best.variant];
        const size_t         groups = ceil_div(rows, static_cast<size_t>(v.block_m))
                              * ceil_div(cols, static_cast<size_t>(v.block_n))
                              * static_cast<size_t>(stream_best.split_k) * batch;
        one_pass = groups <= cus * ((v.block_m == 64 && v.block_n == 64) ? 1 : 2);
    }
    const size_t skinny  = std::min(rows, cols);
    const bool   compete = skinny <= 64 || (skinny <= 128 && one_pass)
                         || (rows * cols <= (size_t{1} << 20) && k <= 4096);
    // (no tiled plan moves A and B faster than operand_bytes_per_us, which is what bounds the
    // skinny shapes; the estimates above rank the tiled plans among themselves without it)
    const double tiled_us = std::max(best, launch_us + operand_us);
    if(have_stream && (!found || (stream_us < tiled_us && compete)))
    {
        *out  = stream_best;
        found = true;
    }
    return found;
}

bool stream_plan(size_t rows, size_t cols, size_t k, bool a_kmajor, bool b_kmajor, size_t batch, size_t cus_of_device,
                 launch_plan* out, double* microseconds)
{
    // skinny, or so small that tiles of 64 x 64 do not outnumber the compute units of an MI355X
    // (K in stages of 128, the last of which may be cut short; rows of a K-contiguous operand
    // must stay 16-byte aligned)
    if(k < 256 || ((a_kmajor || b_kmajor) && k % 8 != 0) || rows == 0 || cols == 0
       || (rows > 128 && cols > 128 && rows * cols > (size_t{1} << 20)))
    {
        return false;
    }
    const model_stream& c      = model_measured.stream;
    const size_t        cus    = cus_of_device != 0 ? cus_of_device : static_cast<size_t>(model_measured.compute_units);
    const size_t        stages = (k + 127) / 128;
    const bool          wide   = cols >= rows; // the large operand is B
    const int           count  = static_cast<int>(sizeof(model_variants) / sizeof(model_variants[0]));
    struct stream_candidate
    {
        double us;
        int    variant, slices;
    };
    constexpr int    max_candidates = 32;
    stream_candidate candidate[max_candidates];
    int              candidates = 0;
    for(int i = 0; i < count; ++i)
    {
        const model_variant& v = model_variants[i];
        if(v.pipeline != 7)
        {
            continue;
        }
        const size_t bm = v.block_m, bn = v.block_n;
        if(bm > 64 || bn > 64)
        {
            continue; // the tiles with a 128-wide side are the tuner's to pick: no constants fitted
        }
        // an operand that is not K-contiguous: k rows of 16-byte pieces; on a 32-wide side of
        // the tile (k rows of 64 bytes, half a cache line a request) only while it is skinny
        // and stays in L2 (1024 x 1024 x 4096 with A column-major: 28.4 us on the 32 x 64
        // tile, 18.6 on 64 x 64)
        if((!a_kmajor && (rows % 8 != 0 || (bm <= 32 && rows > 128)))
           || (!b_kmajor && (cols % 8 != 0 || (bn <= 32 && cols > 128))))
        {
            continue;
        }
        const int    slot    = bm == 16 ? (bn == 64 ? 5 : 4) : bn == 16 ? (bm == 64 ? 7 : 6) : (bm == 64 ? 1 : 0) + (bn == 64 ? 2 : 0);
        const size_t tm      = ceil_div(rows, bm), tn = ceil_div(cols, bn), tiles = tm * tn;
        // (transposing reads: by the width of the side they fill, in units of 64)
        const double other   = (a_kmajor ? 0.0 : static_cast<double>(bm) / 64.0) + (b_kmajor ? 0.0 : static_cast<double>(bn) / 64.0);
        const double per_cu  = c.stage_us[slot] * (1.0 + c.transposed_operand * other);
        const double large   = static_cast<double>(wide ? bn : bm) * 256.0;
        const double small   = static_cast<double>(wide ? bm : bn) * 256.0;
        const double sharing = 1.0 + (static_cast<double>(wide ? tm : tn) - 1.0) * c.panel_sharing;
        const bool   large_kmajor = wide ? b_kmajor : a_kmajor, small_kmajor = wide ? a_kmajor : b_kmajor;
        const double rate    = (large_kmajor ? c.bytes_per_us_kmajor : c.bytes_per_us_other)
                            * (!large_kmajor && (wide ? bn : bm) <= 32 ? c.half_line : 1.0)
                            * (std::max(rows, cols) * k * 2 > (size_t{256} << 20) ? (large_kmajor ? c.beyond_cache : c.beyond_cache_other) : 1.0);
        const double l2_rate = c.bytes_per_us_l2 * (!small_kmajor && (wide ? bm : bn) <= 32 ? c.half_line : 1.0);
        for(size_t s = 1; s <= 8; s *= 2)
        {
            // (the counters of the tiles that several workgroups share: 4096 a launch)
            if(stages % s != 0 || stages / s < 2 || (s > 1 && tiles * batch > 4096))
            {
                continue;
            }
            // (the LDS lets two workgroups run on a compute unit at once, one of the 64 x 64 tile)
            const size_t groups   = tiles * s * batch;
            const size_t resident = cus * ((bm == 64 && bn == 64) ? 1 : 2);
            const double active   = static_cast<double>(groups < resident ? groups : resident);
            const double turns  = 1.0 + static_cast<double>(ceil_div(static_cast<size_t>(active), cus) - 1) * c.taking_turns;
            const double stage  = std::max(per_cu * turns, large * (active / sharing) / rate + small * active / l2_rate);
            const double t      = c.launch_us
                             + static_cast<double>(ceil_div(groups, resident)) * (c.fill_us + static_cast<double>(stages / s) * stage)
                             + (s > 1 ? c.exchange_us + c.exchange_us_per_kb * static_cast<double>(s * bm * bn * 4) / 1024.0 : 0.0);
            if(candidates < max_candidates)
            {
                candidate[candidates++] = {t, i, static_cast<int>(s)};
            }
        }
    }
    if(candidates == 0)
    {
        return false;
    }
    // Of the plans whose estimate is within 3 % of the lowest, the one with the fewest
    // workgroups per tile (the exchange is the least certain part of an estimate), then the
    // lowest: 3.0 -> 2.6 % behind the best timed plan on average over the recorded sweep,
    // 32 -> 20 % at worst.
    double lowest = candidate[0].us;
    for(int j = 1; j < candidates; ++j)
    {
        lowest = std::min(lowest, candidate[j].us);
    }
    const stream_candidate* pick = nullptr;
    for(int j = 0; j < candidates; ++j)
    {
        const stream_candidate& x = candidate[j];
        if(x.us <= lowest * 1.03
           && (pick == nullptr || x.slices < pick->slices || (x.slices == pick->slices && x.us < pick->us)))
        {
            pick = &x;
        }
    }
    *microseconds = pick->us;
    out->variant  = pick->variant;
    out->swizzle  = 1;
    out->split_k  = pick->slices;
    out->touch    = 0;
    return true;
}

launch_plan select_plan_from(const tuned_entry* table, size_t count, size_t m, size_t n, size_t k,
                             int type_idx, int lc, int la, int lb)
{
    const int   group = type_group_of(type_idx);
    launch_plan plan;
    if(find_exact(table, count, m, n, k, group, la, lb, lc, &plan))
    {
        return plan;
    }
    if(group != 0 && find_exact(table, count, m, n, k, 0, la, lb, lc, &plan))
    {
        return plan;
    }
    if(find_closest(table, count, m, n, k, group, la, lb, lc, &plan))
    {
        return plan;
    }
    if(group != 0 && find_closest(table, count, m, n, k, 0, la, lb, lc, &plan))
    {
        return plan;
    }
    return heuristic_plan(m, n, k, lc);
}

namespace
{
// What the whole-K streaming kernel asks of a shape (the pointers are the launch's business):
// a stage of K, 16-byte aligned rows of either kind.
bool streaming_takes(size_t m, size_t n, size_t k, int lc, int la, int lb)
{
    const size_t rows = lc == 0 ? m : n, cols = lc == 0 ? n : m;
    bool         a_kmajor = la == 0, b_kmajor = lb == 1;
    if(lc != 0)
    {
        std::swap(a_kmajor, b_kmajor);
    }
    return k >= 128 && ((!a_kmajor && !b_kmajor) || k % 8 == 0) && (a_kmajor || rows % 8 == 0)
           && (b_kmajor || cols % 8 == 0);
}
} // namespace

launch_plan select_plan(size_t m, size_t n, size_t k, int type_idx, int lc, int la, int lb, size_t batch,
                        size_t cus)
{
    const int   group = type_group_of(type_idx);
    launch_plan plan;
    // the table was tuned on single GEMMs: a batch changes how many tiles there are to
    // spread, which is the model's business
    if(batch > 1 && model_plan(m, n, k, lc, la, lb, &plan, batch, cus))
    {
        return plan;
    }
    // a tuned entry for exactly this shape first (the reference's order, steps 1 and 2) ...
    if(find_exact(tuned_table, tuned_count, m, n, k, group, la, lb, lc, &plan)
       || (group != 0 && find_exact(tuned_table, tuned_count, m, n, k, 0, la, lb, lc, &plan)))
    {
        return plan;
    }
    // ... fewer than 16 rows (or columns) as 16 of them, where that entry runs on the streaming
    // kernel: the tiles, the workgroups and the bytes moved are the same (rows past M are read
    // as zeros), so the plan tuned for 16 is the plan for 1 to 15
    // (8 x 4096 x 14336: 19.9 us on the entry's 32 x 16 tile, 23.6 on the estimate's pick)
    if(std::min(m, n) < 16 && std::max(m, n) >= 512)
    {
        const size_t m16 = std::max<size_t>(m, 16), n16 = std::max<size_t>(n, 16);
        if((find_exact(tuned_table, tuned_count, m16, n16, k, group, la, lb, lc, &plan)
            || (group != 0 && find_exact(tuned_table, tuned_count, m16, n16, k, 0, la, lb, lc, &plan)))
           && model_variants[plan.variant].pipeline == 7 && streaming_takes(m, n, k, lc, la, lb))
        {
            return plan;
        }
    }
    // ... then the model for regular shapes, and the nearest tuned entry for the rest
    if(model_plan(m, n, k, lc, la, lb, &plan, 1, cus))
    {
        return plan;
    }
    // A skinny shape that neither has an entry nor suits the model (rows that are not 16-byte
    // aligned): the nearest tuned entry would be a large square's plan, 256 x 256 tiles
    // for a handful of rows; the shape heuristic cuts K over the compute units instead.
    if(std::min(m, n) <= 64 && std::max(m, n) >= 512)
    {
        return heuristic_plan(m, n, k, lc);
    }
    plan = select_plan_from(tuned_table, tuned_count, m, n, k, type_idx, lc, la, lb);
    // The nearest entry may be a small problem's, tuned onto the streaming kernel, which
    // wants 16-byte aligned rows of either kind: a
    // shape that does not fit takes the shape heuristic's plan instead.
    const model_variant& v = model_variants[plan.variant];
    if(v.pipeline == 7 && !streaming_takes(m, n, k, lc, la, lb))
    {
        return heuristic_plan(m, n, k, lc);
    }
    return plan;
}

} // namespace host
} // namespace rocm_wmma_gemm
