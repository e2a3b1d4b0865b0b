// Cooperative load / store: several waves share the movement of one large fragment.
//
// Same public surface as library/include/rocwmma/rocwmma_coop.hpp:78-412.  A fragment
// is a list of register chunks (internal/layout.hpp); waves [0, waveCount) each take an
// equal contiguous run of chunks.  When waveCount exceeds the number of chunks only the
// first NumChunks waves take part, one chunk each, and the rest return
// (coop_load.hpp:101-131 has the same rule).  A wave keeps its share in the first
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
        // workgroups hold at most 16 waves; counts must be powers of two
        switch(waveCount)
        {
        case 1u: load_matrix_coop_sync<1u>(frag, data, ldm, waveIndex); break;
        case 2u: load_matrix_coop_sync<2u>(frag, data, ldm, waveIndex); break;
        case 4u: load_matrix_coop_sync<4u>(frag, data, ldm, waveIndex); break;
        case 8u: load_matrix_coop_sync<8u>(frag, data, ldm, waveIndex); break;
        case 16u: load_matrix_coop_sync<16u>(frag, data, ldm, waveIndex); break;
        default: break;
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
        switch(waveCount)
        {
        case 1u: store_matrix_coop_sync<1u>(data, frag, ldm, waveIndex); break;
        case 2u: store_matrix_coop_sync<2u>(data, frag, ldm, waveIndex); break;
        case 4u: store_matrix_coop_sync<4u>(data, frag, ldm, waveIndex); break;
        case 8u: store_matrix_coop_sync<8u>(data, frag, ldm, waveIndex); break;
        case 16u: store_matrix_coop_sync<16u>(data, frag, ldm, waveIndex); break;
        default: break;
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
