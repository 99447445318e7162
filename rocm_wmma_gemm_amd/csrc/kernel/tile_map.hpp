// Workgroup id -> output tile, for a chip whose 256 CUs sit in 8 XCDs with one
// L2 each.  The hardware deals consecutive workgroup ids round-robin over the
// XCDs, so ids that are congruent mod 8 share an L2.  The map first renumbers
// the ids so that every XCD owns one contiguous run of "logical" ids, then walks
// the tile grid in bands of `group` tile rows (or columns), column by column inside a band,
// so that a run of logical ids covers a compact group x (run/group) rectangle of
// C and re-uses the same A row panels and B column panels out of that L2.
//
// Plays the role of the reference's tile_mapper (reference
// rocm_wmma_gemm/include/rocm_wmma_gemm/kernel/mapping.hpp:34-324); unlike the
// reference's maps it is a bijection for every grid, with no clamping.
#ifndef ROCM_WMMA_GEMM_TILE_MAP_HPP
#define ROCM_WMMA_GEMM_TILE_MAP_HPP

#if defined(__HIPCC__)
#define RWG_HD __host__ __device__
#else
#define RWG_HD
#endif

namespace rocm_wmma_gemm
{
namespace device
{

constexpr int num_xcd = 8;

struct tile_coord
{
    int m;
    int n;
};

// Contiguous-per-XCD renumbering of [0, total).
RWG_HD inline int xcd_remap(int wg, int total)
{
    const int per_xcd = (total + num_xcd - 1) / num_xcd; // ids owned by a "tall" XCD
    const int rem     = total % num_xcd;
    const int tall    = rem == 0 ? num_xcd : rem; // XCDs that own per_xcd ids
    const int xcd     = wg % num_xcd;
    const int local   = wg / num_xcd;
    if(xcd < tall)
    {
        return xcd * per_xcd + local;
    }
    return tall * per_xcd + (xcd - tall) * (per_xcd - 1) + local;
}

// Banded walk.  group > 0: bands of `group` tile rows; inside a band, down a column
// first.  group < 0: the mirror image, bands of -group tile columns, along a row first
// (a grid that is wider than tall then gives an XCD the rectangle that the upright walk
// gives it on the transposed grid).  group 0 counts as 1.
RWG_HD inline tile_coord banded_tile(int id, int grid_m, int grid_n, int group)
{
    const bool mirrored = group < 0;
    const int  g        = mirrored ? -group : (group == 0 ? 1 : group);
    const int  tall     = mirrored ? grid_n : grid_m; // the dimension the bands cut
    const int  wide     = mirrored ? grid_m : grid_n;
    const int  per_band = g * wide;
    const int  band     = id / per_band;
    const int  first    = band * g;
    const int  rows     = (tall - first) < g ? (tall - first) : g;
    const int  in_band  = id - band * per_band;
    const int  along    = first + in_band % rows;
    const int  across   = in_band / rows;
    tile_coord t;
    t.m = mirrored ? across : along;
    t.n = mirrored ? along : across;
    return t;
}

RWG_HD inline tile_coord map_tile(int wg, int grid_m, int grid_n, int group)
{
    return banded_tile(xcd_remap(wg, grid_m * grid_n), grid_m, grid_n, group);
}

} // namespace device
} // namespace rocm_wmma_gemm

#endif // ROCM_WMMA_GEMM_TILE_MAP_HPP
