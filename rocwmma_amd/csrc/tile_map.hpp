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
    __device__ inline bool tileCoord(uint32_t bid, uint32_t tilesM, uint32_t tilesN, uint32_t& tm, uint32_t& tn)
    {
        constexpr uint32_t XCDS = 8, GROUP_M = 4;
        const uint32_t     total  = tilesM * tilesN;
        const uint32_t     perXcd = (total + XCDS - 1) / XCDS;
        const uint32_t     id     = (bid % XCDS) * perXcd + bid / XCDS;
        if(id >= total)
            return false;
        const uint32_t groupSize = GROUP_M * tilesN;
        const uint32_t group     = id / groupSize;
        const uint32_t first     = group * GROUP_M;
        const uint32_t rowsHere  = (tilesM - first) < GROUP_M ? (tilesM - first) : GROUP_M;
        const uint32_t inGroup   = id % groupSize;
        tm                       = first + inGroup % rowsHere;
        tn                       = inGroup / rowsHere;
        return true;
    }

} // namespace r355

#endif // R355_TILE_MAP_HPP
