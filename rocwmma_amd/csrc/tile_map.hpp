// Workgroup-id to output-tile mapping shared by the macro-tile kernels.
#ifndef R355_TILE_MAP_HPP
#define R355_TILE_MAP_HPP

#include <cstdint>

#include <hip/hip_runtime.h>

namespace r355
{
    // Workgroup id -> (tile row, tile col).  Hardware deals workgroup ids round-robin to the
    // 8 XCDs; ids with the same (id mod 8) share an L2.  Give each XCD a contiguous run of
    // tile indices and walk the run in groups of GROUP_M tile rows, column by column, so that
    // the 32 tiles resident on an XCD at one time cover about 4 x 8 tiles.
    __device__ inline void tileOfId(uint32_t id, uint32_t tilesM, uint32_t tilesN, uint32_t& tm, uint32_t& tn)
    {
        constexpr uint32_t GROUP_M   = 4;
        const uint32_t     groupSize = GROUP_M * tilesN;
        const uint32_t     group     = id / groupSize;
        const uint32_t     first     = group * GROUP_M;
        const uint32_t     rowsHere  = (tilesM - first) < GROUP_M ? (tilesM - first) : GROUP_M;
        const uint32_t     inGroup   = id % groupSize;
        tm                           = first + inGroup % rowsHere;
        tn                           = inGroup / rowsHere;
    }

    __device__ inline bool tileCoord(uint32_t bid, uint32_t tilesM, uint32_t tilesN, uint32_t& tm, uint32_t& tn)
    {
        constexpr uint32_t XCDS   = 8;
        const uint32_t     total  = tilesM * tilesN;
        const uint32_t     perXcd = (total + XCDS - 1) / XCDS;
        const uint32_t     id     = (bid % XCDS) * perXcd + bid / XCDS;
        if(id >= total)
            return false;
        tileOfId(id, tilesM, tilesN, tm, tn);
        return true;
    }

    // A launch that covers only the tile indices [first, first + count) of the walk above (the same split of the
    // run over the XCDs).  With `quad` the indices name tiles of twice the edge - tilesM x tilesN is then the grid
    // of those - and every index is covered by four workgroups of the same XCD; tm, tn come back in units of the
    // launch's own (half-edge) tiles and may lie outside the matrix for a partial last row or column of tiles.
    __device__ inline bool tileCoordRange(uint32_t bid, uint32_t tilesM, uint32_t tilesN, uint32_t first, uint32_t count,
                                          bool quad, uint32_t& tm, uint32_t& tn)
    {
        constexpr uint32_t XCDS   = 8;
        const uint32_t     perXcd = (count + XCDS - 1) / XCDS;
        const uint32_t     slot   = quad ? bid / (4u * XCDS) : bid / XCDS; // position in the XCD's run
        const uint32_t     local  = (bid % XCDS) * perXcd + slot;
        if(slot >= perXcd || local >= count)
            return false;
        tileOfId(first + local, tilesM, tilesN, tm, tn);
        if(quad)
        {
            const uint32_t sub = (bid / XCDS) % 4u;
            tm                 = 2u * tm + sub / 2u;
            tn                 = 2u * tn + sub % 2u;
        }
        return true;
    }

} // namespace r355

#endif // R355_TILE_MAP_HPP
