// Stand-alone I/O arithmetic of a BlockDim x BlockK block moved by one wave with VectorWidth elements
// per lane and operation (public name and enumerators of the reference's io_traits.hpp:43-82).
// Fragments carry the same facts for their own layout in IOConfig<...>::IOTraits.
#ifndef ROCWMMA_IO_TRAITS_HPP
#define ROCWMMA_IO_TRAITS_HPP

#include "constants.hpp"
#include "types.hpp"
#include "utils.hpp"

namespace rocwmma
{
    template <uint32_t BlockDim, uint32_t BlockK, typename DataT, uint32_t VectorWidth = 1>
    struct IOTraits
    {
        enum : uint32_t
        {
            ThreadsPerIO  = Constants::AMDGCN_WAVE_SIZE, // lanes taking part in one operation
            ElementsPerIO = ThreadsPerIO * VectorWidth, // elements one operation moves
            KPerIO        = (ElementsPerIO + BlockDim - 1u) / BlockDim, // BlockDim-strides per operation
            ElementCount  = BlockDim * BlockK, // elements of the whole block
            IOCount       = (ElementCount + ElementsPerIO - 1u) / ElementsPerIO, // operations per block
            // per-lane storage: one slot per element, or per 32-bit register
            UnpackedSize = (ElementCount + ThreadsPerIO - 1u) / ThreadsPerIO,
            PackedSize   = (UnpackedSize + PackTraits<DataT>::PackRatio - 1u) / PackTraits<DataT>::PackRatio,
            // hardware registers holding the block
            PackedVRegCount   = ElementCount * sizeof(DataT) / Constants::AMDGCN_REGISTER_SIZE_BYTES,
            UnpackedVRegCount = PackedVRegCount * PackTraits<DataT>::PackRatio
        };

        static_assert(ElementCount % ElementsPerIO == 0u, "the block does not split into equal wave-wide operations");
        static_assert(ElementCount % ThreadsPerIO == 0u, "the block does not split evenly over the lanes of a wave");
        static_assert(BlockDim <= ElementsPerIO ? (ElementsPerIO % BlockDim == 0u || ElementsPerIO % BlockK == 0u)
                                                : (BlockDim % ElementsPerIO == 0u || BlockK % ElementsPerIO == 0u),
                      "one operation must cover whole BlockDim strides, or a whole fraction of one");
    };
} // namespace rocwmma

#endif // ROCWMMA_IO_TRAITS_HPP
