// Implementation of the shape -> launch plan lookup (plain C++, no device code).
#include "config_select.hpp"

#include <limits>

#include "config_generated.hpp"

namespace rocm_wmma_gemm
{
namespace host
{

const tuned_entry* const tuned_table = generated::entries;
const size_t             tuned_count = generated::entry_count;

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

launch_plan select_plan(size_t m, size_t n, size_t k, int type_idx, int lc, int la, int lb)
{
    return select_plan_from(tuned_table, tuned_count, m, n, k, type_idx, lc, la, lb);
}

} // namespace host
} // namespace rocm_wmma_gemm
