// Fragment <-> memory movement for one wave (and for a share of a cooperative fragment).
//
// Reference counterparts: opaque_load.hpp:59-140, opaque_store.hpp:57-134 (whole
// fragment per wave) and coop_load.hpp:107-218, coop_store.hpp:108-222 (stride space
// split over waves).  Here a fragment is a list of register chunks (KW consecutive
// KDim elements each, see layout.hpp); a chunk moves as one vector access when KDim is
// the contiguous memory dimension and as KW element accesses, coalesced across lanes,
// otherwise.  Pointers may be global or LDS; vector accesses need the natural
// alignment of KW elements, as the reference's vector-width accesses do.
#ifndef ROCWMMA_IO_HPP
#define ROCWMMA_IO_HPP

#include "layout.hpp"

namespace rocwmma
{
    namespace detail
    {
        template <typename DataT, uint32_t N>
        struct alignas(sizeof(DataT) * N) Packet
        {
            DataT v[N];
        };

        template <typename MatrixT,
                  uint32_t BlockM,
                  uint32_t BlockN,
                  uint32_t BlockK,
                  typename DataT,
                  typename DataLayoutT>
        struct FragmentIO
        {
            using Layout = RegisterLayout<MatrixT, BlockM, BlockN, BlockK, DataT>;
            using Map1d  = DataSpace<DataLayoutT>;

            static constexpr uint32_t KW         = Layout::KW;
            static constexpr bool     Contiguous = kContiguous_v<MatrixT, DataLayoutT>;

            ROCWMMA_DEVICE static inline uint32_t lane()
            {
                // blockDim.x is a multiple of 64 (mapping_util.hpp), so this is the hardware lane
                return threadIdx.x % Constants::AMDGCN_WAVE_SIZE_64;
            }

            // offset of (BlockDim index d, KDim index k)
            ROCWMMA_DEVICE static inline uint32_t offset(uint32_t d, uint32_t k, uint32_t ldm)
            {
                return Map1d::fromMatrixCoord(Layout::matrixCoord(d, k), ldm);
            }

            // Chunks [FirstChunk, FirstChunk + Count) of memory <-> registers [RegChunk...)
            template <uint32_t Count>
            ROCWMMA_DEVICE static inline void
                load(DataT* regs, DataT const* data, uint32_t ldm, uint32_t firstChunk)
            {
                const uint32_t l = lane();
#pragma unroll
                for(uint32_t c = 0; c < Count; ++c)
                {
                    const uint32_t d = Layout::dimOf(l, firstChunk + c);
                    const uint32_t k = Layout::kOf(l, firstChunk + c);
                    if constexpr(Contiguous)
                    {
                        using P = Packet<DataT, KW>;
                        *reinterpret_cast<P*>(regs + c * KW)
                            = *reinterpret_cast<P const*>(data + offset(d, k, ldm));
                    }
                    else
                    {
                        const uint32_t base = offset(d, k, ldm);
#pragma unroll
                        for(uint32_t e = 0; e < KW; ++e)
                            regs[c * KW + e] = data[base + e * ldm];
                    }
                }
            }

            template <uint32_t Count>
            ROCWMMA_DEVICE static inline void
                store(DataT* data, DataT const* regs, uint32_t ldm, uint32_t firstChunk)
            {
                const uint32_t l = lane();
#pragma unroll
                for(uint32_t c = 0; c < Count; ++c)
                {
                    const uint32_t d = Layout::dimOf(l, firstChunk + c);
                    const uint32_t k = Layout::kOf(l, firstChunk + c);
                    if constexpr(Contiguous)
                    {
                        using P = Packet<DataT, KW>;
                        *reinterpret_cast<P*>(data + offset(d, k, ldm))
                            = *reinterpret_cast<P const*>(regs + c * KW);
                    }
                    else
                    {
                        const uint32_t base = offset(d, k, ldm);
#pragma unroll
                        for(uint32_t e = 0; e < KW; ++e)
                            data[base + e * ldm] = regs[c * KW + e];
                    }
                }
            }
        };
    } // namespace detail
} // namespace rocwmma

#endif // ROCWMMA_IO_HPP
