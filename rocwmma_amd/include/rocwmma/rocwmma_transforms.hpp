// Fragment type transforms: transpose and data-layout change.
//
// Same public surface as library/include/rocwmma/rocwmma_transforms.hpp:36-66.  In the
// reference a data-layout change may need a cross-lane AOS<->SOA shuffle
// (rocwmma_transforms_impl.hpp:181-270).  Here register layouts never depend on the
// memory orientation and A / B layouts mirror each other (internal/layout.hpp), so both
// transforms only relabel the fragment type: the registers are returned unchanged.
//   transpose : fragment<matrix_a, M, N, K, T, L>  <->  fragment<matrix_b, N, M, K, T, orthogonal(L)>
//               (matrix_a and matrix_b only, as in the reference)
#ifndef ROCWMMA_TRANSFORMS_API_HPP
#define ROCWMMA_TRANSFORMS_API_HPP

#include "rocwmma.hpp"

namespace rocwmma
{
    namespace detail
    {
        template <typename FragT>
        struct ApplyTranspose;

        template <uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT, typename DataLayoutT>
        struct ApplyTranspose<fragment<matrix_a, BlockM, BlockN, BlockK, DataT, DataLayoutT>>
        {
            using Type
                = fragment<matrix_b, BlockN, BlockM, BlockK, DataT, orthogonal_layout_t<DataLayoutT>>;
        };

        template <uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT, typename DataLayoutT>
        struct ApplyTranspose<fragment<matrix_b, BlockM, BlockN, BlockK, DataT, DataLayoutT>>
        {
            using Type
                = fragment<matrix_a, BlockN, BlockM, BlockK, DataT, orthogonal_layout_t<DataLayoutT>>;
        };

        template <typename FragT, typename NewDataLayoutT>
        struct ApplyDataLayout;

        template <typename MatrixT,
                  uint32_t BlockM,
                  uint32_t BlockN,
                  uint32_t BlockK,
                  typename DataT,
                  typename DataLayoutT,
                  typename NewDataLayoutT>
        struct ApplyDataLayout<fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>, NewDataLayoutT>
        {
            using Type = fragment<MatrixT, BlockM, BlockN, BlockK, DataT, NewDataLayoutT>;
        };

        template <typename FragT>
        struct ApplyRegisterFile;

        template <typename MatrixT,
                  uint32_t BlockM,
                  uint32_t BlockN,
                  uint32_t BlockK,
                  typename DataT,
                  typename DataLayoutT>
        struct ApplyRegisterFile<fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>>
        {
            using FragT = fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>;
            // BlockDim = wave size, KDim = elements per lane
            using Type = fragment<matrix_b, 1u, Constants::AMDGCN_WAVE_SIZE_64, FragT::num_elements, DataT, row_major>;
        };

        // Same registers under another fragment type, preserving const / reference category
        template <typename ToFragT, typename FromFragT>
        ROCWMMA_DEVICE inline decltype(auto) relabel(FromFragT&& frag)
        {
            using From = std::remove_reference_t<FromFragT>;
            static_assert(sizeof(ToFragT) == sizeof(std::decay_t<FromFragT>),
                          "fragment relabel must keep the register footprint");
            if constexpr(std::is_lvalue_reference_v<FromFragT>)
            {
                if constexpr(std::is_const_v<From>)
                    return reinterpret_cast<ToFragT const&>(frag);
                else
                    return reinterpret_cast<ToFragT&>(frag);
            }
            else
            {
                ToFragT out;
                out.mStorage = reinterpret_cast<ToFragT const&>(frag).mStorage;
                return out;
            }
        }
    } // namespace detail

    template <typename FragT>
    using ApplyTranspose_t = typename detail::ApplyTranspose<std::decay_t<FragT>>::Type;

    template <typename FragT, typename NewDataLayoutT>
    using ApplyDataLayout_t = typename detail::ApplyDataLayout<std::decay_t<FragT>, NewDataLayoutT>::Type;

    template <typename FragT>
    using ApplyRegisterFile_t = typename detail::ApplyRegisterFile<std::decay_t<FragT>>::Type;

    template <typename FragT>
    ROCWMMA_DEVICE static inline decltype(auto) applyTranspose(FragT&& frag)
    {
        return detail::relabel<ApplyTranspose_t<FragT>>(static_cast<FragT&&>(frag));
    }

    template <typename DataLayoutT, uint32_t WaveCount = 1, typename FragT>
    ROCWMMA_DEVICE static inline decltype(auto) applyDataLayout(FragT&& frag)
    {
        return detail::relabel<ApplyDataLayout_t<FragT, DataLayoutT>>(static_cast<FragT&&>(frag));
    }

} // namespace rocwmma

#endif // ROCWMMA_TRANSFORMS_API_HPP
