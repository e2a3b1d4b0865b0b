// Wave-level matrix fragment API for gfx950 (MI355X).
//
// Same public surface as library/include/rocwmma/rocwmma.hpp:127-316 of the reference:
// fragment<>, fill_fragment, load_matrix_sync, store_matrix_sync, mma_sync,
// synchronize_workgroup.  Every call is collective over the 64 lanes of a wave.
// Register layouts are the gfx950 MFMA operand layouts (internal/layout.hpp), so
// mma_sync is a straight sequence of matrix instructions with no data movement.
#ifndef ROCWMMA_API_HPP
#define ROCWMMA_API_HPP

#include "internal/config.hpp"
#include "internal/constants.hpp"
#include "internal/convert.hpp"
#include "internal/flow_control.hpp"
#include "internal/io.hpp"
#include "internal/io_traits.hpp"
#include "internal/layout.hpp"
#include "internal/mapping_util.hpp"
#include "internal/mfma.hpp"
#include "internal/type_traits.hpp"
#include "internal/types.hpp"
#include "internal/utils.hpp"

namespace rocwmma
{
    // Compile-time description of a fragment; the names samples and tests reach through the
    // accessor aliases below.  Reference: io_config.hpp:65-113, io_shape.hpp:43-80,
    // io_traits.hpp:43-82.
    template <typename MatrixT,
              uint32_t BlockM,
              uint32_t BlockN,
              uint32_t BlockK,
              typename DataT,
              typename DataLayoutT>
    struct IOConfig
    {
        using RegLayout = detail::RegisterLayout<MatrixT, BlockM, BlockN, BlockK, DataT>;

        struct IOShape
        {
            enum : uint32_t
            {
                BlockHeight = RegLayout::BlockHeight,
                BlockWidth  = RegLayout::BlockWidth,
                BlockDim    = RegLayout::BlockDim,
                KDim        = RegLayout::KDim,
            };
        };

        struct IOTraits
        {
            enum : uint32_t
            {
                ThreadsPerIO     = Constants::AMDGCN_WAVE_SIZE_64,
                ElementsPerIO    = Constants::AMDGCN_WAVE_SIZE_64 * RegLayout::KW,
                KPerIO           = RegLayout::ChunkK,
                ElementCount     = RegLayout::BlockDim * RegLayout::KDim,
                IOCount          = RegLayout::NumChunks,
                UnpackedSize     = RegLayout::NumElements,
                PackedSize       = RegLayout::NumElements * sizeof(DataT) / 4u,
                UnpackedVRegCount = UnpackedSize,
                PackedVRegCount   = PackedSize,
            };
        };

        using IOLayout   = RegLayout;
        using DataLayout = detail::DataSpace<DataLayoutT>;
        using MappingUtil
            = rocwmma::MappingUtil<IOShape::BlockHeight, IOShape::BlockWidth, DataT, DataLayoutT>;
    };

    template <typename MatrixT,
              uint32_t BlockM,
              uint32_t BlockN,
              uint32_t BlockK,
              typename DataT,
              typename DataLayoutT = void>
    class __align__(4) fragment
    {
    public:
        using IOConfigT = IOConfig<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>;
        using IOTraits  = typename IOConfigT::IOTraits;

        struct Traits
        {
            // One 32-bit register lane per packed element: float for f32 data, int otherwise
            using PackedElementT
                = std::conditional_t<std::is_same_v<DataT, float32_t>, float32_t, int32_t>;
            using StorageT = detail::vec_t<PackedElementT, IOTraits::PackedSize>;
            constexpr static uint32_t Size = IOTraits::UnpackedSize;
        };

        // Contents are undefined until filled or loaded
        ROCWMMA_DEVICE fragment() {}
        ROCWMMA_DEVICE fragment(const fragment& other)
        {
            mStorage = other.mStorage;
        }
        ROCWMMA_DEVICE fragment& operator=(const fragment& other)
        {
            mStorage = other.mStorage;
            return *this;
        }

        ROCWMMA_DEVICE inline DataT& operator[](uint32_t index)
        {
            return x[index];
        }
        ROCWMMA_DEVICE inline DataT const& operator[](uint32_t index) const
        {
            return x[index];
        }
        ROCWMMA_DEVICE inline typename Traits::StorageT& operator*()
        {
            return mStorage;
        }
        ROCWMMA_DEVICE inline typename Traits::StorageT const& operator*() const
        {
            return mStorage;
        }

        ROCWMMA_DEVICE constexpr static inline uint32_t height()
        {
            return IOConfigT::IOShape::BlockHeight;
        }
        ROCWMMA_DEVICE constexpr static inline uint32_t width()
        {
            return IOConfigT::IOShape::BlockWidth;
        }
        ROCWMMA_DEVICE constexpr static inline uint32_t blockDim()
        {
            return IOConfigT::IOShape::BlockDim;
        }
        ROCWMMA_DEVICE constexpr static inline uint32_t kDim()
        {
            return IOConfigT::IOShape::KDim;
        }
        ROCWMMA_DEVICE constexpr static inline uint32_t size()
        {
            return num_elements;
        }

        union
        {
            typename Traits::StorageT mStorage; // packed 32-bit registers
            DataT                     x[Traits::Size]; // element view of the same registers
        };
        static_assert(sizeof(typename Traits::StorageT) == sizeof(DataT) * Traits::Size,
                      "Storage and element views must cover the same registers");

        constexpr static uint32_t num_elements = Traits::Size;
        using element_type                     = DataT;
    };

    // ---------------------------------------------------------------- accessors
    // Reference: accessors.hpp:35-89, accessors_impl.hpp:52-130.
    namespace detail
    {
        template <typename FragT>
        struct FragmentTraits;

        template <typename MatrixT_,
                  uint32_t BlockM_,
                  uint32_t BlockN_,
                  uint32_t BlockK_,
                  typename DataT_,
                  typename DataLayoutT_>
        struct FragmentTraits<fragment<MatrixT_, BlockM_, BlockN_, BlockK_, DataT_, DataLayoutT_>>
        {
            using MatrixT     = MatrixT_;
            using DataT       = DataT_;
            using DataLayoutT = DataLayoutT_;
            static constexpr uint32_t BlockM = BlockM_;
            static constexpr uint32_t BlockN = BlockN_;
            static constexpr uint32_t BlockK = BlockK_;
            using IOConfigT = IOConfig<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>;
        };
    } // namespace detail

    template <typename FragT>
    using GetIOConfig_t = typename detail::FragmentTraits<std::decay_t<FragT>>::IOConfigT;
    // Cooperative configuration: the register layout does not depend on how many waves share the
    // fragment (waves take whole register chunks), so WaveCount only parameterises the name
    // (reference: coop_io_config.hpp:63-108, accessors_impl.hpp:99-112).
    template <typename FragT, uint32_t WaveCount = 1u>
    using GetCoopIOConfig_t = GetIOConfig_t<FragT>;
    template <typename FragT>
    using GetIOShape_t = typename GetIOConfig_t<FragT>::IOShape;
    template <typename FragT>
    using GetIOTraits_t = typename GetIOConfig_t<FragT>::IOTraits;
    template <typename FragT>
    using GetDataType_t = typename detail::FragmentTraits<std::decay_t<FragT>>::DataT;
    template <typename FragT>
    using GetDataLayout_t = typename GetIOConfig_t<FragT>::DataLayout;
    template <typename FragT>
    using GetMappingUtil_t = typename GetIOConfig_t<FragT>::MappingUtil;

    // ---------------------------------------------------------------- fill
    template <typename MatrixT,
              uint32_t BlockM,
              uint32_t BlockN,
              uint32_t BlockK,
              typename DataT,
              typename DataLayoutT>
    ROCWMMA_DEVICE inline void
        fill_fragment(fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>& frag, DataT value)
    {
        using FragT = fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>;
#pragma unroll
        for(uint32_t i = 0; i < FragT::num_elements; ++i)
            frag.x[i] = value;
    }

    // ---------------------------------------------------------------- load
    template <typename MatrixT,
              uint32_t BlockM,
              uint32_t BlockN,
              uint32_t BlockK,
              typename DataT,
              typename DataLayoutT>
    ROCWMMA_DEVICE inline void
        load_matrix_sync(fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>& frag,
                         const DataT*                                                   data,
                         uint32_t                                                       ldm)
    {
        static_assert(!std::is_same_v<DataLayoutT, void>,
                      "Must provide layout information. Either statically assign data layout in "
                      "fragment declaration or use the run-time function overload.");
        using IO = detail::FragmentIO<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>;
        IO::template load<IO::Layout::NumChunks>(frag.x, data, ldm, 0u);
    }

    template <typename MatrixT, uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT>
    ROCWMMA_DEVICE inline void
        load_matrix_sync(fragment<MatrixT, BlockM, BlockN, BlockK, DataT>& frag,
                         const DataT*                                      data,
                         uint32_t                                          ldm,
                         layout_t                                          layout)
    {
        // The register layout does not depend on the memory orientation, so the untyped
        // fragment is the same registers as either typed one.
        using FragRowMajor = fragment<MatrixT, BlockM, BlockN, BlockK, DataT, row_major>;
        using FragColMajor = fragment<MatrixT, BlockM, BlockN, BlockK, DataT, col_major>;
        if(layout == layout_t::mem_row_major)
            load_matrix_sync(reinterpret_cast<FragRowMajor&>(frag), data, ldm);
        else
            load_matrix_sync(reinterpret_cast<FragColMajor&>(frag), data, ldm);
    }

    // ---------------------------------------------------------------- store
    template <typename MatrixT,
              uint32_t BlockM,
              uint32_t BlockN,
              uint32_t BlockK,
              typename DataT,
              typename DataLayoutT>
    ROCWMMA_DEVICE inline void
        store_matrix_sync(DataT*                                                               data,
                          fragment<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT> const& frag,
                          uint32_t                                                             ldm)
    {
        static_assert(!std::is_same_v<DataLayoutT, void>,
                      "Must provide data layout. Either statically assign data layout in "
                      "fragment declaration or use the run-time function overload.");
        using IO = detail::FragmentIO<MatrixT, BlockM, BlockN, BlockK, DataT, DataLayoutT>;
        IO::template store<IO::Layout::NumChunks>(data, frag.x, ldm, 0u);
    }

    template <typename MatrixT, uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT>
    ROCWMMA_DEVICE inline void
        store_matrix_sync(DataT*                                                  data,
                          fragment<MatrixT, BlockM, BlockN, BlockK, DataT> const& frag,
                          uint32_t                                                ldm,
                          layout_t                                                layout)
    {
        using FragRowMajor = fragment<MatrixT, BlockM, BlockN, BlockK, DataT, row_major>;
        using FragColMajor = fragment<MatrixT, BlockM, BlockN, BlockK, DataT, col_major>;
        if(layout == layout_t::mem_row_major)
            store_matrix_sync(data, reinterpret_cast<FragRowMajor const&>(frag), ldm);
        else
            store_matrix_sync(data, reinterpret_cast<FragColMajor const&>(frag), ldm);
    }

    // ---------------------------------------------------------------- mma
    // D = A * B + C on one BlockM x BlockN x BlockK tile; d may alias c.
    // Reference: rocwmma_impl.hpp:314-364.
    template <uint32_t BlockM,
              uint32_t BlockN,
              uint32_t BlockK,
              typename InputT,
              typename ComputeT,
              typename LayoutA,
              typename LayoutB,
              typename LayoutC,
              typename LayoutD>
    ROCWMMA_DEVICE inline void
        mma_sync(fragment<accumulator, BlockM, BlockN, BlockK, ComputeT, LayoutD>&       d,
                 fragment<matrix_a, BlockM, BlockN, BlockK, InputT, LayoutA> const&      a,
                 fragment<matrix_b, BlockM, BlockN, BlockK, InputT, LayoutB> const&      b,
                 fragment<accumulator, BlockM, BlockN, BlockK, ComputeT, LayoutC> const& c)
    {
        static_assert(BlockM == BlockN && (BlockM == 16u || BlockM == 32u),
                      "mma_sync supports 16x16 and 32x32 blocks");
        using LayoutAReg = detail::RegisterLayout<matrix_a, BlockM, BlockN, BlockK, InputT>;
        using LayoutBReg = detail::RegisterLayout<matrix_b, BlockM, BlockN, BlockK, InputT>;
        static_assert(LayoutAReg::KW == LayoutBReg::KW && LayoutAReg::NumChunks == LayoutBReg::NumChunks,
                      "A and B register layouts must mirror each other");
        using Op   = detail::MfmaChunk<InputT, BlockM, LayoutAReg::KW>;
        using AccT = typename Op::AccT;
        using AccE = std::conditional_t<detail::is_i8_v<InputT>,
                                        int32_t,
                                        std::conditional_t<std::is_same_v<InputT, float64_t>, float64_t, float32_t>>;
        constexpr uint32_t AccN = BlockM == 32u ? 16u : 4u;

        AccT acc;
        if constexpr(std::is_same_v<ComputeT, AccE>)
        {
            __builtin_memcpy(&acc, c.x, sizeof(AccT));
        }
        else
        {
            // 16-bit compute types: the matrix core accumulates in f32 (mfma_impl.hpp:81-114)
#pragma unroll
            for(uint32_t i = 0; i < AccN; ++i)
                acc[i] = convert<AccE>(c.x[i]);
        }

#pragma unroll
        for(uint32_t chunk = 0; chunk < LayoutAReg::NumChunks; ++chunk)
            Op::exec(acc, a.x + chunk * LayoutAReg::KW, b.x + chunk * LayoutAReg::KW);

        if constexpr(std::is_same_v<ComputeT, AccE>)
        {
            __builtin_memcpy(d.x, &acc, sizeof(AccT));
        }
        else
        {
#pragma unroll
            for(uint32_t i = 0; i < AccN; ++i)
                d.x[i] = convert<ComputeT>(static_cast<AccE>(acc[i]));
        }
    }

    // Workgroup barrier; needed around LDS hand-offs between waves.
    ROCWMMA_DEVICE inline void synchronize_workgroup()
    {
        __syncthreads();
    }

} // namespace rocwmma

#endif // ROCWMMA_API_HPP
