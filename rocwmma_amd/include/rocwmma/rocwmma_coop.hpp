// Cooperative load / store: several waves share the movement of one large fragment.
//
// Same public surface as library/include/rocwmma/rocwmma_coop.hpp:78-412.  A fragment
// is a list of register chunks (internal/layout.hpp); waves [0, waveCount) each take an
// equal contiguous run of chunks.  When waveCount exceeds the number of chunks only the
// first NumChunks waves take part, one chunk each, and the rest return
// (coop_load.hpp:101-131 has the same rule); a run-time waveCount that is not a power of two is
// rounded down to one and the surplus waves return.  A wave keeps its share in the first
// registers of its fragment, so a cooperatively loaded fragment is meaningful only to a
// cooperative store with identical (waveIndex, waveCount).  waveIndex must be uniform
// over the wave.  Hand-offs through LDS need synchronize_workgroup() around them.
#ifndef ROCWMMA_COOP_API_HPP
#define ROCWMMA_COOP_API_HPP

#include "rocwmma.hpp"

namespace rocwmma
{
    namespace detail
    {
        template <uint32_t WaveCount, uint32_t NumChunks>
        struct CoopSplit
        {
            static_assert(isPow2(WaveCount), "WaveCount must be a power of two");
            static_assert(isPow2(NumChunks), "fragment chunk count must be a power of two");
            static constexpr uint32_t ActiveWaves   = cmin(WaveCount, NumChunks);
            static constexpr uint32_t ChunksPerWave = NumChunks / ActiveWaves;
        };

        // Waves that share the work for a wave count given at run time: the largest power of two that does not
        // exceed it (at most 16, a workgroup's maximum; a count of 0 is taken as 1).  Chunk counts are powers of two,
        // so this count either divides the chunks or exceeds them (CoopSplit then lets one wave per chunk take part).
        // Waves with waveIndex at or above it return without touching their fragment, so a workgroup of 3, 6 or 12
        // waves still moves the whole fragment.  (The reference halves the given count until it divides its work
        // items, coop_load.hpp:101-104 -- 6 waves become 3 and then 1; either way every element moves exactly once
        // and the surplus waves idle.)
        ROCWMMA_HOST_DEVICE constexpr inline uint32_t coopWaves(uint32_t waveCount)
        {
            return waveCount >= 16u ? 16u : (waveCount >= 8u ? 8u : (waveCount >= 4u ? 4u : (waveCount >= 2u ? 2u : 1u)));
        }
    } // namespace detail

    template <uint32_t WaveCount,
              typename MatrixT,
              uint32_t BlockM,
              uint32_t BlockN,
              uint32_t BlockK,
              typename DataT,
              typename DataLayoutT>
    ROCWMMA_DEVICE inline void
        load_matrix_coop_sync(fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>& frag,
                              const DataT*                                                   data,
                              uint32_t                                                       ldm,
                              uint32_t                                                       waveIndex)
    {
        using IO    = detail::FragmentIO<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>;
        using Split = detail::CoopSplit<WaveCount, IO::Layout::NumChunks>;
#if ROCWMMA_DEVICE_COMPILE
        waveIndex = __builtin_amdgcn_readfirstlane(waveIndex);
#endif
        if(waveIndex >= Split::ActiveWaves)
            return;
        IO::template load<Split::ChunksPerWave>(frag.x, data, ldm, waveIndex * Split::ChunksPerWave);
    }

    template <uint32_t WaveCount,
              typename MatrixT,
              uint32_t BlockM,
              uint32_t BlockN,
              uint32_t BlockK,
              typename DataT,
              typename DataLayoutT>
    ROCWMMA_DEVICE inline void store_matrix_coop_sync(
        DataT*                                                               data,
        fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT> const& frag,
        uint32_t                                                             ldm,
        uint32_t                                                             waveIndex)
    {
        using IO    = detail::FragmentIO<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>;
        using Split = detail::CoopSplit<WaveCount, IO::Layout::NumChunks>;
#if ROCWMMA_DEVICE_COMPILE
        waveIndex = __builtin_amdgcn_readfirstlane(waveIndex);
#endif
        if(waveIndex >= Split::ActiveWaves)
            return;
        IO::template store<Split::ChunksPerWave>(data, frag.x, ldm, waveIndex * Split::ChunksPerWave);
    }

    // Runtime wave count
    template <typename MatrixT,
              uint32_t BlockM,
              uint32_t BlockN,
              uint32_t BlockK,
              typename DataT,
              typename DataLayoutT>
    ROCWMMA_DEVICE inline void
        load_matrix_coop_sync(fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>& frag,
                              const DataT*                                                   data,
                              uint32_t                                                       ldm,
                              uint32_t                                                       waveIndex,
                              uint32_t                                                       waveCount)
    {
        // workgroups hold at most 16 waves
        switch(detail::coopWaves(waveCount))
        {
        case 1u: load_matrix_coop_sync<1u>(frag, data, ldm, waveIndex); break;
        case 2u: load_matrix_coop_sync<2u>(frag, data, ldm, waveIndex); break;
        case 4u: load_matrix_coop_sync<4u>(frag, data, ldm, waveIndex); break;
        case 8u: load_matrix_coop_sync<8u>(frag, data, ldm, waveIndex); break;
        default: load_matrix_coop_sync<16u>(frag, data, ldm, waveIndex); break;
        }
    }

    template <typename MatrixT,
              uint32_t BlockM,
              uint32_t BlockN,
              uint32_t BlockK,
              typename DataT,
              typename DataLayoutT>
    ROCWMMA_DEVICE inline void store_matrix_coop_sync(
        DataT*                                                               data,
        fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT> const& frag,
        uint32_t                                                             ldm,
        uint32_t                                                             waveIndex,
        uint32_t                                                             waveCount)
    {
        switch(detail::coopWaves(waveCount))
        {
        case 1u: store_matrix_coop_sync<1u>(data, frag, ldm, waveIndex); break;
        case 2u: store_matrix_coop_sync<2u>(data, frag, ldm, waveIndex); break;
        case 4u: store_matrix_coop_sync<4u>(data, frag, ldm, waveIndex); break;
        case 8u: store_matrix_coop_sync<8u>(data, frag, ldm, waveIndex); break;
        default: store_matrix_coop_sync<16u>(data, frag, ldm, waveIndex); break;
        }
    }

    // All waves of the workgroup, in row-major wave order (rocwmma_coop_impl.hpp:98-107)
    template <typename MatrixT,
              uint32_t BlockM,
              uint32_t BlockN,
              uint32_t BlockK,
              typename DataT,
              typename DataLayoutT>
    ROCWMMA_DEVICE inline void
        load_matrix_coop_sync(fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>& frag,
                              const DataT*                                                   data,
                              uint32_t                                                       ldm)
    {
        using Mapping  = GetMappingUtil_t<std::decay_t<decltype(frag)>>;
        auto waveCoord = Mapping::waveCoord();
        auto wgDim     = Mapping::workgroupDim();
        load_matrix_coop_sync(frag,
                              data,
                              ldm,
                              get<0>(waveCoord) * get<1>(wgDim) + get<1>(waveCoord),
                              get<0>(wgDim) * get<1>(wgDim));
    }

    template <typename MatrixT,
              uint32_t BlockM,
              uint32_t BlockN,
              uint32_t BlockK,
              typename DataT,
              typename DataLayoutT>
    ROCWMMA_DEVICE inline void store_matrix_coop_sync(
        DataT*                                                               data,
        fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT> const& frag,
        uint32_t                                                             ldm)
    {
        using Mapping  = GetMappingUtil_t<std::decay_t<decltype(frag)>>;
        auto waveCoord = Mapping::waveCoord();
        auto wgDim     = Mapping::workgroupDim();
        store_matrix_coop_sync(data,
                               frag,
                               ldm,
                               get<0>(waveCoord) * get<1>(wgDim) + get<1>(waveCoord),
                               get<0>(wgDim) * get<1>(wgDim));
    }

    // Deprecated split-count forms: the split count no longer has an effect
    template <uint32_t WaveCount,
              uint32_t SplitCount,
              typename MatrixT,
              uint32_t BlockM,
              uint32_t BlockN,
              uint32_t BlockK,
              typename DataT,
              typename DataLayoutT>
    [[deprecated("SplitCount argument is deprecated")]] ROCWMMA_DEVICE inline void
        load_matrix_coop_sync(fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>& frag,
                              const DataT*                                                   data,
                              uint32_t                                                       ldm,
                              uint32_t                                                       waveIndex)
    {
        load_matrix_coop_sync<WaveCount>(frag, data, ldm, waveIndex);
    }

    template <uint32_t WaveCount,
              uint32_t SplitCount,
              typename MatrixT,
              uint32_t BlockM,
              uint32_t BlockN,
              uint32_t BlockK,
              typename DataT,
              typename DataLayoutT>
    [[deprecated("SplitCount argument is deprecated")]] ROCWMMA_DEVICE inline void
        store_matrix_coop_sync(
            DataT*                                                               data,
            fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT> const& frag,
            uint32_t                                                             ldm,
            uint32_t                                                             waveIndex)
    {
        store_matrix_coop_sync<WaveCount>(data, frag, ldm, waveIndex);
    }

    template <typename MatrixT,
              uint32_t BlockM,
              uint32_t BlockN,
              uint32_t BlockK,
              typename DataT,
              typename DataLayoutT>
    [[deprecated("splitCount argument is deprecated")]] ROCWMMA_DEVICE inline void
        load_matrix_coop_sync(fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>& frag,
                              const DataT*                                                   data,
                              uint32_t                                                       ldm,
                              uint32_t                                                       waveIndex,
                              uint32_t                                                       waveCount,
                              uint32_t /*splitCount*/)
    {
        load_matrix_coop_sync(frag, data, ldm, waveIndex, waveCount);
    }

    template <typename MatrixT,
              uint32_t BlockM,
              uint32_t BlockN,
              uint32_t BlockK,
              typename DataT,
              typename DataLayoutT>
    [[deprecated("splitCount argument is deprecated")]] ROCWMMA_DEVICE inline void
        store_matrix_coop_sync(
            DataT*                                                               data,
            fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT> const& frag,
            uint32_t                                                             ldm,
            uint32_t                                                             waveIndex,
            uint32_t                                                             waveCount,
            uint32_t /*splitCount*/)
    {
        store_matrix_coop_sync(data, frag, ldm, waveIndex, waveCount);
    }

} // namespace rocwmma

#endif // ROCWMMA_COOP_API_HPP
