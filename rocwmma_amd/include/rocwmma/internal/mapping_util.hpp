// Wave / block / matrix coordinate helpers for kernels that give each wave one block.
// Same interface as library/include/rocwmma/internal/mapping_util.hpp:42-206.  Assumes
// blockDim = (wavesX * 64, wavesY): the wave coordinate is (threadIdx.x / 64, threadIdx.y).
#ifndef ROCWMMA_MAPPING_UTIL_HPP
#define ROCWMMA_MAPPING_UTIL_HPP

#include "layout.hpp"

namespace rocwmma
{
    namespace detail
    {
        template <uint32_t TBlockX = 0u, uint32_t TBlockY = 0u>
        struct WaveSpace
        {
            using WaveCoordT      = Coord2d;
            using WorkgroupCoordT = Coord2d;
            using WorkgroupDimT   = Coord2d;

            ROCWMMA_DEVICE static inline uint32_t localLaneId()
            {
                return threadIdx.x % Constants::AMDGCN_WAVE_SIZE;
            }
            ROCWMMA_DEVICE static inline WaveCoordT localWaveCoord()
            {
                return make_coord2d(threadIdx.x / Constants::AMDGCN_WAVE_SIZE, threadIdx.y);
            }
            // Compile-time constant when the workgroup shape is given as template arguments
            ROCWMMA_DEVICE constexpr static inline WorkgroupDimT workgroupDim()
            {
                if constexpr(TBlockX > 0u && TBlockY > 0u)
                    return make_coord2d(TBlockX / Constants::AMDGCN_WAVE_SIZE, TBlockY);
                else
                    return make_coord2d(blockDim.x / Constants::AMDGCN_WAVE_SIZE, blockDim.y);
            }
            ROCWMMA_DEVICE static inline WorkgroupCoordT workgroupCoord()
            {
                return make_coord2d(blockIdx.x, blockIdx.y);
            }
            ROCWMMA_DEVICE static inline WaveCoordT globalWaveCoord()
            {
                return workgroupCoord() * workgroupDim() + localWaveCoord();
            }
        };

        template <uint32_t BlockHeight, uint32_t BlockWidth>
        struct MatrixSpace
        {
            using MatrixCoordT = Coord2d;
            using BlockCoordT  = Coord2d;

            ROCWMMA_HOST_DEVICE constexpr static inline MatrixCoordT
                fromBlockCoord(BlockCoordT const& blockCoord)
            {
                return make_coord2d(get<0>(blockCoord) * BlockHeight, get<1>(blockCoord) * BlockWidth);
            }
        };
    } // namespace detail

    template <uint32_t BlockHeight, uint32_t BlockWidth, typename DataT, typename DataLayout>
    struct MappingUtil
    {
        using WaveSpace   = detail::WaveSpace<>;
        using MatrixSpace = detail::MatrixSpace<BlockHeight, BlockWidth>;
        using DataSpace   = detail::DataSpace<DataLayout>;

        using WaveCoordT    = typename WaveSpace::WaveCoordT;
        using BlockCoordT   = typename MatrixSpace::BlockCoordT;
        using MatrixCoordT  = typename MatrixSpace::MatrixCoordT;
        using WorkgroupDimT = typename WaveSpace::WorkgroupDimT;

        ROCWMMA_DEVICE static inline uint32_t laneId()
        {
            return WaveSpace::localLaneId();
        }
        // Local wave coordinate relative to the workgroup
        ROCWMMA_DEVICE static inline WaveCoordT waveCoord()
        {
            return WaveSpace::localWaveCoord();
        }
        // Global block (grid) coordinate of the current wave
        ROCWMMA_DEVICE static inline BlockCoordT blockCoord()
        {
            return WaveSpace::globalWaveCoord();
        }
        // Matrix coordinate of the current wave's block
        ROCWMMA_DEVICE static inline MatrixCoordT matrixCoord()
        {
            return MatrixSpace::fromBlockCoord(blockCoord());
        }
        ROCWMMA_DEVICE static inline DataT const* dataCoord(DataT const* baseAddr, uint32_t ldm)
        {
            return baseAddr + DataSpace::fromMatrixCoord(matrixCoord(), ldm);
        }
        ROCWMMA_DEVICE static inline DataT* dataCoord(DataT* baseAddr, uint32_t ldm)
        {
            return baseAddr + DataSpace::fromMatrixCoord(matrixCoord(), ldm);
        }
        ROCWMMA_DEVICE static inline WorkgroupDimT workgroupDim()
        {
            return WaveSpace::workgroupDim();
        }

        // Coordinate overrides
        ROCWMMA_DEVICE static inline BlockCoordT blockCoordM(uint32_t m)
        {
            auto c  = blockCoord();
            get<0>(c) = m;
            return c;
        }
        ROCWMMA_DEVICE static inline BlockCoordT blockCoordN(uint32_t n)
        {
            auto c  = blockCoord();
            get<1>(c) = n;
            return c;
        }
        ROCWMMA_DEVICE static inline MatrixCoordT matrixCoordM(uint32_t m)
        {
            auto c  = matrixCoord();
            get<0>(c) = m;
            return c;
        }
        ROCWMMA_DEVICE static inline MatrixCoordT matrixCoordN(uint32_t n)
        {
            auto c  = matrixCoord();
            get<1>(c) = n;
            return c;
        }

        // Conversions
        ROCWMMA_DEVICE static inline MatrixCoordT matrixCoord(BlockCoordT const& blockCoord)
        {
            return MatrixSpace::fromBlockCoord(blockCoord);
        }
        ROCWMMA_DEVICE static inline uint32_t dataOffset(MatrixCoordT const& matrixCoord, uint32_t ldm)
        {
            return DataSpace::fromMatrixCoord(matrixCoord, ldm);
        }
        ROCWMMA_DEVICE static inline DataT const*
            dataCoord(DataT const* baseAddr, MatrixCoordT const& matrixCoord, uint32_t ldm)
        {
            return baseAddr + DataSpace::fromMatrixCoord(matrixCoord, ldm);
        }
        ROCWMMA_DEVICE static inline DataT*
            dataCoord(DataT* baseAddr, MatrixCoordT const& matrixCoord, uint32_t ldm)
        {
            return baseAddr + DataSpace::fromMatrixCoord(matrixCoord, ldm);
        }
    };
} // namespace rocwmma

#endif // ROCWMMA_MAPPING_UTIL_HPP
