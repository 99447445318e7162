// Host-only checks of the pieces of the library that need no GPU: the tile map
// (compiled here for the CPU) and the config selection functions.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <set>
#include <utility>
#include <vector>

#include "config_select.hpp"
#include "kernel/tile_map.hpp"
#include "workspace_policy.hpp"

using namespace rocm_wmma_gemm::device;
using namespace rocm_wmma_gemm::host;

static int fail(const char* what)
{
    std::printf("FAIL: %s\n", what);
    return 1;
}

static int check_tilemap()
{
    const int groups[] = {0, 1, 2, 4, 8, 16, 100, -1, -2, -4, -8, -16, -100}; // negative: bands of tile columns
    for(int gm = 1; gm <= 40; ++gm)
        for(int gn = 1; gn <= 40; ++gn)
            for(int g : groups)
            {
                std::set<std::pair<int, int>> seen;
                for(int wg = 0; wg < gm * gn; ++wg)
                {
                    tile_coord t = map_tile(wg, gm, gn, g);
                    if(t.m < 0 || t.m >= gm || t.n < 0 || t.n >= gn)
                        return fail("tile outside grid");
                    if(!seen.insert({t.m, t.n}).second)
                        return fail("tile visited twice");
                }
            }
    // xcd_remap alone is a permutation for any total
    for(int total = 1; total <= 300; ++total)
    {
        std::vector<int> hit(total, 0);
        for(int wg = 0; wg < total; ++wg)
        {
            int id = xcd_remap(wg, total);
            if(id < 0 || id >= total || hit[id]++)
                return fail("xcd_remap not a permutation");
        }
    }
    std::printf("tilemap ok\n");
    return 0;
}

static int check_xcd()
{
    // 16 x 16 tiles, band height 4: the 32 workgroups of one XCD (ids = xcd mod 8)
    // must cover a 4 x 8 rectangle: 4 distinct tile rows, 8 distinct tile columns.
    for(int xcd = 0; xcd < 8; ++xcd)
    {
        std::set<int> rows, cols;
        for(int wg = xcd; wg < 256; wg += 8)
        {
            tile_coord t = map_tile(wg, 16, 16, 4);
            rows.insert(t.m);
            cols.insert(t.n);
        }
        if(rows.size() != 4 || cols.size() != 8)
            return fail("XCD footprint is not a 4x8 rectangle");
    }
    // mirrored walk (negative group): on a 16 x 32 grid with bands of 4 tile columns an
    // XCD's 64 tiles cover what the upright walk gives it on the 32 x 16 grid, transposed
    for(int wg = 0; wg < 512; ++wg)
    {
        const tile_coord a = map_tile(wg, 16, 32, -4), b = map_tile(wg, 32, 16, 4);
        if(a.m != b.n || a.n != b.m)
            return fail("mirrored walk is not the transpose of the upright walk");
    }
    std::printf("xcd ok\n");
    return 0;
}

static int check_select()
{
    // layouts: la, lb, lc ; plan {variant, swizzle, split_k}
    const tuned_entry table[] = {
        {1024, 1024, 1024, 0, 0, 1, 0, {1, 4, 1}},
        {2048, 2048, 2048, 0, 0, 1, 0, {2, 8, 1}},
        {65536, 2048, 2048, 0, 0, 1, 0, {3, 8, 1}},
        {4096, 4096, 4096, 0, 0, 1, 0, {4, 16, 1}},
        {4096, 4096, 4096, 1, 0, 1, 0, {5, 16, 1}},
        {4096, 16384, 4096, 0, 0, 1, 0, {6, 16, 1}},
        {512, 512, 512, 0, 1, 1, 1, {7, 4, 2}},
    };
    const size_t n = sizeof(table) / sizeof(table[0]);
    auto pick = [&](size_t m, size_t nn, size_t k, int type_idx, int lc, int la, int lb) {
        return select_plan_from(table, n, m, nn, k, type_idx, lc, la, lb).variant;
    };
    // exact hit, 16-bit group
    if(pick(4096, 4096, 4096, 0, 0, 0, 1) != 4)
        return fail("exact hit");
    // exact hit in the fp32 group wins over group 0
    if(pick(4096, 4096, 4096, 1, 0, 0, 1) != 5)
        return fail("group-1 exact hit");
    // fp32 group without its own exact entry falls back to group 0's exact entry
    if(pick(2048, 2048, 2048, 3, 0, 0, 1) != 2)
        return fail("group-1 -> group-0 exact fallback");
    // nearest K first (2048), then nearest (M, N): (2048,2048) beats (65536,2048)
    if(pick(8192, 4096, 2048, 0, 0, 0, 1) != 2)
        return fail("closest: K first then MN");
    // K = 4096 group: (4096,14336) is nearer to (4096,16384) than to (4096,4096)
    if(pick(4096, 14336, 4096, 0, 0, 0, 1) != 6)
        return fail("closest: MN distance");
    // a genuine hit on the LAST entry is honoured (no sentinel collision)
    if(pick(512, 512, 512, 0, 1, 1, 1) != 7)
        return fail("hit on last entry");
    // layout triple with no entries at all -> heuristic (variant 0 or 1)
    launch_plan h = select_plan_from(table, n, 300, 300, 300, 0, 1, 0, 0);
    if(h.variant != 0 || h.split_k != 1)
        return fail("heuristic for uncovered layout");
    // heuristic: few tiles and long K -> split-K
    launch_plan lk = heuristic_plan(1024, 1024, 65536, 0);
    if(lk.split_k < 2)
        return fail("heuristic split-K on long K");
    // empty table
    launch_plan e = select_plan_from(nullptr, 0, 4096, 4096, 4096, 0, 0, 0, 1);
    if(e.variant != 1)
        return fail("heuristic on empty table");
    // The model for regular shapes without a tuned entry: what matters is how the tile
    // count falls on 256 CUs.
    struct tile { int bm, bn, pipeline; };
#define RWG_VARIANT(IDX, BM, BN, BK, WM, WN, PIPE) {BM, BN, PIPE},
    const tile tiles[] = {
#include "variants.def"
    };
#undef RWG_VARIANT
    launch_plan p;
    // 3584^3: 196 tiles of 256 x 256 in one wave, not 361 of 192 x 192 in two
    if(!model_plan(3584, 3584, 3584, 0, 0, 1, &p) || tiles[p.variant].bm != 256 || tiles[p.variant].bn != 256
       || tiles[p.variant].pipeline != 5 || p.split_k != 1)
        return fail("model: 3584^3");
    // 3072^3, both operands K-contiguous: 256 tiles of 192 x 192
    if(!model_plan(3072, 3072, 3072, 0, 0, 1, &p) || tiles[p.variant].bm != 192 || tiles[p.variant].bn != 192)
        return fail("model: 3072^3");
    // the same with both operands M/N-contiguous: 192-wide tiles are not built
    if(!model_plan(3072, 3072, 3072, 0, 1, 0, &p) || tiles[p.variant].bm % 128 != 0
       || tiles[p.variant].bn % 128 != 0)
        return fail("model: 3072^3, transposed operands");
    // a column-major C swaps the operands: A row-major, B row-major, C column-major has
    // kernel-space A = B^T (M/N-contiguous), B = A^T (K-contiguous)
    if(!model_plan(3072, 3072, 3072, 1, 0, 0, &p) || tiles[p.variant].bm % 128 != 0)
        return fail("model: operand swap under a column-major C");
    // few tiles, long K: some split
    if(!model_plan(304, 4096, 4096, 0, 0, 1, &p) || p.split_k == 1)
        return fail("model: 304 x 4096 x 4096 wants a split");
    if(!model_plan(1024, 1024, 65536, 0, 0, 1, &p) || p.split_k == 1)
        return fail("model: long K wants a split");
    // decode-like shapes: the whole-K streaming kernel, 64 rows of the large operand per
    // workgroup when it has 8192 of them, also when a column-major C swaps the operands
    if(!model_plan(32, 8192, 8192, 0, 0, 1, &p) || tiles[p.variant].pipeline != 7 || tiles[p.variant].bm != 32
       || tiles[p.variant].bn != 64 || p.split_k != 1)
        return fail("model: skinny M streams");
    if(!model_plan(32, 8192, 8192, 1, 0, 1, &p) || tiles[p.variant].pipeline != 7 || tiles[p.variant].bm != 64
       || tiles[p.variant].bn != 32)
        return fail("model: skinny M under a column-major C streams as skinny N");
    if(!model_plan(32, 8192, 8192, 0, 0, 0, &p) || tiles[p.variant].pipeline != 7 || tiles[p.variant].bn != 64)
        return fail("model: weights stored K x N stream on the 64-wide side");
    // the large operand, when it is not K-contiguous, sits on a 64-wide side of the tile (whole
    // cache lines); the small one may sit on a 32-wide side
    if(!model_plan(32, 8192, 8192, 0, 1, 1, &p) || tiles[p.variant].pipeline != 7 || tiles[p.variant].bm != 32
       || tiles[p.variant].bn != 64)
        return fail("model: activations stored K x M stream on the 32-wide side");
    if(!model_plan(32, 8192, 8192, 0, 1, 0, &p) || tiles[p.variant].pipeline != 7 || tiles[p.variant].bn != 64)
        return fail("model: weights stored K x N next to activations stored K x M stream on the 64-wide side");
    // few tiles and a long K: several workgroups per tile
    if(!model_plan(16, 1024, 8192, 0, 0, 1, &p) || tiles[p.variant].pipeline != 7 || p.split_k < 2)
        return fail("model: 32 tiles of a skinny shape are shared between workgroups");
    // fewer than 16 rows, or rows that are no multiple of 8: the streaming kernel alone
    if(!model_plan(8, 4096, 4096, 0, 0, 1, &p) || tiles[p.variant].pipeline != 7)
        return fail("model: 8 rows stream");
    if(!model_plan(3, 4096, 4096, 0, 0, 1, &p) || tiles[p.variant].pipeline != 7)
        return fail("model: 3 rows stream");
    if(model_plan(3, 4096, 4096, 0, 1, 1, &p))
        return fail("model: 3 rows that are not K-contiguous are nobody's");
    if(!model_plan(128, 28672, 8192, 0, 0, 1, &p) || tiles[p.variant].pipeline == 7)
        return fail("model: 128 rows against a very large operand stay with the tiled kernels");
    if(!model_plan(256, 8192, 8192, 0, 0, 1, &p) || tiles[p.variant].pipeline == 7)
        return fail("model: 256 rows are not skinny");
    // 65 to 128 rows: in every layout, while the streaming plan's workgroups all run at once
    if(!model_plan(128, 4096, 4096, 0, 0, 1, &p) || tiles[p.variant].pipeline != 7)
        return fail("model: 128 rows against 4096 x 4096, both K-contiguous, stream");
    if(!model_plan(128, 4096, 4096, 0, 1, 0, &p) || tiles[p.variant].pipeline != 7)
        return fail("model: 128 rows against 4096 x 4096, neither K-contiguous, stream");
    if(!model_plan(128, 14336, 4096, 0, 0, 1, &p) || tiles[p.variant].pipeline == 7)
        return fail("model: 128 rows against 14336 x 4096 (two passes of streaming workgroups) stay with the tiled kernels");
    // a large operand past the memory-side cache (470 MB): streamed when it is K-contiguous
    // (the tiled kernels do not move operands faster than operand_bytes_per_us), left to the
    // tiled kernels' split along K when it is not
    if(!model_plan(16, 28672, 8192, 0, 0, 1, &p) || tiles[p.variant].pipeline != 7 || p.split_k != 1)
        return fail("model: 16 rows against 28672 x 8192, K-contiguous, stream");
    if(!model_plan(16, 28672, 8192, 0, 0, 0, &p) || tiles[p.variant].pipeline == 7)
        return fail("model: 16 rows against 8192 x 28672 stored row-major stay with the tiled kernels");
    // small problems: at most 2^20 elements of C, any layout
    if(!model_plan(512, 2048, 2048, 0, 0, 0, &p) || tiles[p.variant].pipeline != 7)
        return fail("model: 512 x 2048 x 2048 streams");
    if(!model_plan(512, 2048, 2048, 0, 1, 0, &p) || tiles[p.variant].pipeline != 7)
        return fail("model: 512 x 2048 x 2048 with neither operand K-contiguous streams");
    if(!model_plan(2048, 1024, 1024, 0, 0, 1, &p) || tiles[p.variant].pipeline == 7)
        return fail("model: 2048 x 1024 x 1024 is too large for a workgroup per small tile");
    // a skinny shape the model does not take (K-contiguous rows of 4001 elements) and the
    // table does not hold: the shape heuristic's split, not the nearest large square's plan
    {
        const launch_plan q = select_plan(8, 4096, 4001, 0, 0, 0, 1);
        if(tiles[q.variant].pipeline != 0 || q.split_k < 2)
            return fail("select: skinny shape with K = 4001");
    }
    // fewer than 16 rows take the plan tuned for 16 rows of the same N, K and layouts when it
    // is the streaming kernel's (and the shape suits that kernel)
    {
        const launch_plan q16 = select_plan(16, 4096, 14336, 0, 0, 0, 1), q3 = select_plan(3, 4096, 14336, 0, 0, 0, 1);
        if(tiles[q16.variant].pipeline != 7 || q3.variant != q16.variant || q3.split_k != q16.split_k)
            return fail("select: 3 rows take the plan of the tuned 16 rows");
        // (the model alone would send 3 rows elsewhere: that is what the entry is for)
        launch_plan by_model;
        if(model_plan(3, 4096, 14336, 0, 0, 1, &by_model) && by_model.variant == q16.variant && by_model.split_k == q16.split_k)
            return fail("select: the check above needs a shape where entry and estimate differ");
        // A stored K x M with 3 rows: k rows of 6 bytes, not the streaming kernel's
        const launch_plan r3 = select_plan(3, 4096, 14336, 0, 0, 1, 1);
        if(tiles[r3.variant].pipeline == 7)
            return fail("select: 3 rows that are not K-contiguous must not stream");
    }
    // next to 1024^3, whose entries run on the streaming kernel: K-contiguous rows that are
    // not 16-byte aligned must not inherit that plan
    {
        const launch_plan q = select_plan(81, 1132, 1274, 0, 0, 0, 1);
        if(tiles[q.variant].pipeline == 7)
            return fail("select: the streaming kernel's plan for rows it cannot take");
    }
    // K in stages of 128 of which the last is cut short
    if(!model_plan(16, 4096, 1000, 0, 0, 1, &p) || tiles[p.variant].pipeline != 7)
        return fail("model: a skinny shape with K = 1000 streams");
    // 272 tiles of 256 x 256: the last wave of 16 tiles split
    if(!model_plan(4352, 4096, 8192, 0, 0, 1, &p) || tiles[p.variant].pipeline != 5 || p.split_k >= -1)
        return fail("model: tail split");
    // a partial last K tile with aligned rows: the persistent kernel takes it as it is,
    // every other kernel would pay padded copies of both operands
    // 400 tiles: the 144 tiles of the tail wave cut in two would be 288 slices, two more
    // passes over the CUs for what one pass of whole tiles does (measured 0.255 ms against
    // 0.210 ms whole)
    if(!model_plan(5120, 5120, 5120, 0, 0, 1, &p) || p.split_k != 1)
        return fail("model: a tail wave whose slices need two passes stays whole");
    if(!model_plan(4096, 4096, 1000, 0, 0, 1, &p) || tiles[p.variant].pipeline != 5)
        return fail("model: ragged K with aligned rows belongs to the persistent kernel");
    // K-contiguous rows that are not 16-byte aligned, odd extents: not its business ...
    if(model_plan(4096, 4096, 1001, 0, 0, 1, &p) || model_plan(4095, 4096, 4096, 0, 0, 1, &p))
        return fail("model must leave irregular shapes alone");
    // ... but an odd K is fine when no operand is K-contiguous (A column-major, B row-major)
    if(!model_plan(4096, 4096, 1001, 0, 1, 0, &p) || tiles[p.variant].pipeline != 5)
        return fail("model: odd K, no K-contiguous operand");
    // another compute-unit count (a partitioned GPU): what fills 256 units in one pass takes
    // passes on fewer, and a shape with too few tiles for 256 has enough for 64
    if(!model_plan(4096, 4096, 4096, 0, 0, 1, &p, 1, 64) || tiles[p.variant].pipeline != 5 || p.split_k != 1)
        return fail("model: 4096^3 on 64 compute units is four whole passes");
    if(!model_plan(2048, 2048, 8192, 0, 0, 1, &p, 1, 256) || tiles[p.variant].bm != 128 || tiles[p.variant].bn != 128)
        return fail("model: 2048 x 2048 on 256 compute units takes the tile that gives 256 tiles");
    if(!model_plan(2048, 2048, 8192, 0, 0, 1, &p, 1, 32) || tiles[p.variant].bm != 256 || p.split_k != 1)
        return fail("model: 2048 x 2048 on 32 compute units takes the large tile, two whole passes");
    if(model_measured.compute_units != 256 || model_measured.step_count < 4)
        return fail("model constants of the generated header");
    std::printf("select ok\n");
    return 0;
}

// The scratch-buffer rules: nothing allocates, frees or synchronises for a call on a
// capturing stream, and a buffer such a call has used is never freed.
static int check_workspace()
{
    using A            = workspace_action;
    const size_t MiB   = size_t{1} << 20;
    const size_t limit = size_t{16} << 30;
    struct
    {
        size_t have, need;
        bool   capturing, lent;
        A      want;
        const char* what;
    } cases[] = {
        {0, 4 * MiB, false, false, A::allocate, "first eager call allocates"},
        {0, 4 * MiB, true, false, A::refuse, "first call under capture gets nothing"},
        {256 * MiB, 4 * MiB, false, false, A::use_existing, "fits, eager"},
        {256 * MiB, 4 * MiB, true, false, A::use_existing, "fits, capturing"},
        {256 * MiB, 256 * MiB, true, true, A::use_existing, "fits exactly"},
        {256 * MiB, 300 * MiB, true, false, A::refuse, "too small under capture: no growth"},
        {256 * MiB, 300 * MiB, true, true, A::refuse, "too small under capture, lent before"},
        {256 * MiB, 300 * MiB, false, false, A::grow_free_old, "eager growth frees the old buffer"},
        {256 * MiB, 300 * MiB, false, true, A::grow_retire_old, "a buffer a graph may hold is kept"},
        {256 * MiB, limit + 1, false, false, A::refuse, "beyond the limit"},
        {0, limit + 1, false, false, A::refuse, "beyond the limit, nothing there"},
        {0, 0, false, false, A::allocate, "a zero-byte request still gets a buffer"},
    };
    for(const auto& c : cases)
    {
        if(workspace_decide(c.have, c.need, limit, c.capturing, c.lent) != c.want)
            return fail(c.what);
    }
    // whatever the state, a capturing stream never triggers an allocation or a free
    for(size_t have : {size_t{0}, MiB, 256 * MiB})
        for(size_t need : {size_t{1}, MiB, 257 * MiB})
            for(bool lent : {false, true})
            {
                const A a = workspace_decide(have, need, limit, true, lent);
                if(a != A::use_existing && a != A::refuse)
                    return fail("capture must not allocate or free");
                if(a == A::use_existing && have < need)
                    return fail("handed out a buffer that is too small");
            }
    if(workspace_grown_size(4 * MiB, 256 * MiB) != 256 * MiB || workspace_grown_size(400 * MiB, 256 * MiB) != 500 * MiB)
        return fail("grown size");
    std::printf("workspace ok\n");
    return 0;
}

// The model's plan for one problem, for tests that compare it with measurements:
//   host_checks model M N K lc la lb [batch [compute units]]
// prints "variant swizzle split touch block_m block_n block_k waves_m waves_n pipeline", or "none".
static int print_model(int argc, char** argv)
{
    if(argc < 8)
        return 2;
    struct tile { int bm, bn, bk, wm, wn, pipeline; };
#define RWG_VARIANT(IDX, BM, BN, BK, WM, WN, PIPE) {BM, BN, BK, WM, WN, PIPE},
    const tile tiles[] = {
#include "variants.def"
    };
#undef RWG_VARIANT
    const size_t m = std::strtoull(argv[2], nullptr, 10), n = std::strtoull(argv[3], nullptr, 10),
                 k = std::strtoull(argv[4], nullptr, 10);
    const int    lc = std::atoi(argv[5]), la = std::atoi(argv[6]), lb = std::atoi(argv[7]);
    const size_t batch = argc > 8 ? std::strtoull(argv[8], nullptr, 10) : 1;
    const size_t cus   = argc > 9 ? std::strtoull(argv[9], nullptr, 10) : 0;
    launch_plan  p;
    if(!model_plan(m, n, k, lc, la, lb, &p, batch, cus))
    {
        std::printf("none\n");
        return 0;
    }
    const tile& t = tiles[p.variant];
    std::printf("%d %d %d %d %d %d %d %d %d %d\n", p.variant, p.swizzle, p.split_k, p.touch, t.bm, t.bn, t.bk, t.wm,
                t.wn, t.pipeline);
    return 0;
}

// "stream rows cols k a_kmajor b_kmajor": the streaming kernel's cheapest plan by estimate,
// as "block_m block_n workgroups_per_tile microseconds", or "none".
static int print_stream(int argc, char** argv)
{
    if(argc < 7)
        return 2;
    struct tile { int bm, bn, bk, wm, wn, pipeline; };
#define RWG_VARIANT(IDX, BM, BN, BK, WM, WN, PIPE) {BM, BN, BK, WM, WN, PIPE},
    const tile tiles[] = {
#include "variants.def"
    };
#undef RWG_VARIANT
    const size_t rows = std::strtoull(argv[2], nullptr, 10), cols = std::strtoull(argv[3], nullptr, 10),
                 k = std::strtoull(argv[4], nullptr, 10);
    launch_plan p;
    double      us = 0.0;
    if(!stream_plan(rows, cols, k, std::atoi(argv[5]) != 0, std::atoi(argv[6]) != 0, 1, 0, &p, &us))
    {
        std::printf("none\n");
        return 0;
    }
    std::printf("%d %d %d %.6f\n", tiles[p.variant].bm, tiles[p.variant].bn, p.split_k, us);
    return 0;
}

int main(int argc, char** argv)
{
    if(argc < 2)
        return 2;
    if(!std::strcmp(argv[1], "model"))
        return print_model(argc, argv);
    if(!std::strcmp(argv[1], "stream"))
        return print_stream(argc, argv);
    if(!std::strcmp(argv[1], "tilemap"))
        return check_tilemap();
    if(!std::strcmp(argv[1], "xcd"))
        return check_xcd();
    if(!std::strcmp(argv[1], "select"))
        return check_select();
    if(!std::strcmp(argv[1], "workspace"))
        return check_workspace();
    return 2;
}
