// 2:4 structured-sparse fragments on the gfx950 sparse matrix cores (v_smfmac_*).
//
// The reference has no sparse path; this header extends its fragment API
// (library/include/rocwmma/rocwmma.hpp:127-202 fragment, :300-313 mma_sync) with
//   fragment<sparse_matrix_a, BlockM, BlockN, BlockK, DataT, row_major>   the kept half of a BlockM x BlockK block of A
//   fragment<sparse_metadata, BlockM, BlockN, BlockK, DataT>              their 2-bit positions, one register per instruction
//   load_matrix_sync(fragA, values, ldStage), load_matrix_sync(fragMeta, meta, ldStage)
//   mma_sync(d, fragA, fragMeta, fragB, c)                                 d = A * B + c with a dense matrix_b fragment
// A keeps 2 of every aligned group of 4 elements along k.  B is an ordinary matrix_b fragment of the same block
// shape: the sparse instructions read B in the register layout of the dense double-K instructions (a lane holds
// 16 consecutive bytes of K per 64-byte half step), which is what matrix_b fragments of 8- and 16-bit types
// already are.  Accumulators are ordinary accumulator fragments.
//
// Operand formats as measured on MI355X with one-hot A against coded B (16 x 16 x 128 int8 and 16 x 16 x 64 f16;
// the 32 x 32 shapes follow the same rule with two lane groups):
//   * A: lane l holds 16 bytes of kept elements of row l % D: those of the dense elements
//     [(l / D) * S / G, (l / D + 1) * S / G) of the instruction's S-wide K step, in order (D = block edge, G = 64 / D);
//   * index register: bits [2 p + 1 : 2 p] = position within its group of 4 of the lane's kept element p
//     (16-bit types: 8 kept elements, the low 16 bits, ABID 0);
//   * B: lane l holds bytes [16 (l / D), 16 (l / D) + 16) of each half of the step's K bytes of column l % D.
//
// Storage ("K-blocked": everything one K stage of a run of rows needs is contiguous, so that a macro tile's
// stage is one linear copy and a fragment's 16 bytes per lane are consecutive across lanes).  With ES the
// element size, a stage is 128 dense bytes of K = 128 / ES elements, and m the number of rows of A (m % 16 == 0,
// k % (128 / ES) == 0):
//   values  [stage][row / 16][lane group g = 0..3][row % 16][16 bytes]
//           the kept elements of dense k in [stage * 128 / ES + g * 32 / ES, ... + 32 / ES) of that row, in order
//   meta    the same indexing with 4 / ES bytes per (stage, row, g): one nibble idx0 | idx1 << 2 (idx0 < idx1) per
//           group of 4, the lane's first group in the lowest bits -- the word is the index register as it is
#ifndef ROCWMMA_SPARSE_API_HPP
#define ROCWMMA_SPARSE_API_HPP

#include "rocwmma.hpp"

namespace rocwmma
{
    // fragment roles
    struct sparse_matrix_a
    {
    };
    struct sparse_metadata
    {
    };

    // Where things are in the K-blocked storage of a 2:4 sparse m x k matrix of DataT
    template <typename DataT>
    struct Sparse24
    {
        static constexpr uint32_t ES         = sizeof(DataT);
        static constexpr uint32_t StageK     = 128u / ES; // dense elements of k per stage
        static constexpr uint32_t ChunkElems = 16u / ES; // kept elements per lane per instruction
        static constexpr uint32_t MetaBytes  = 4u / ES; // index bytes per lane per instruction

        // elements (values) / bytes (meta) between consecutive K stages
        ROCWMMA_HOST_DEVICE constexpr static inline uint32_t valueStageStride(uint32_t m)
        {
            return m * (64u / ES);
        }
        ROCWMMA_HOST_DEVICE constexpr static inline uint32_t metaStageStride(uint32_t m)
        {
            return m * (16u / ES);
        }
        // offset of the block that starts at (row, k): row % 16 == 0, k % StageK == 0
        ROCWMMA_HOST_DEVICE constexpr static inline uint64_t valueOffset(uint32_t row, uint32_t k, uint32_t m)
        {
            return (uint64_t)(k / StageK) * valueStageStride(m) + (uint64_t)(row / 16u) * (1024u / ES);
        }
        ROCWMMA_HOST_DEVICE constexpr static inline uint64_t metaOffset(uint32_t row, uint32_t k, uint32_t m)
        {
            return (uint64_t)(k / StageK) * metaStageStride(m) + (uint64_t)(row / 16u) * (256u / ES);
        }
        // byte offsets inside a stage of (row, lane group g)
        ROCWMMA_HOST_DEVICE constexpr static inline uint32_t valueByteInStage(uint32_t row, uint32_t g)
        {
            return (row / 16u) * 1024u + g * 256u + (row % 16u) * 16u;
        }
        ROCWMMA_HOST_DEVICE constexpr static inline uint32_t metaByteInStage(uint32_t row, uint32_t g)
        {
            return ((row / 16u) * 64u + g * 16u + (row % 16u)) * MetaBytes;
        }
    };

    namespace detail
    {
        template <uint32_t BlockM, uint32_t BlockK, typename DataT>
        struct SparseShape
        {
            static_assert(BlockM == 16u || BlockM == 32u, "sparse blocks are 16 or 32 rows");
            static_assert(sizeof(DataT) == 1u || sizeof(DataT) == 2u, "sparse matrix instructions take 8- and 16-bit elements");
            static constexpr uint32_t ES     = sizeof(DataT);
            static constexpr uint32_t G      = 64u / BlockM; // lane groups along k
            static constexpr uint32_t StepK  = (BlockM == 16u ? 128u : 64u) / ES; // dense k per instruction
            static constexpr uint32_t Steps  = BlockK / StepK;
            static constexpr uint32_t PerLane = 16u / ES; // kept elements per lane per instruction
            static_assert(BlockK % Sparse24<DataT>::StageK == 0u, "sparse fragments cover whole 128-byte K stages");
        };
    } // namespace detail

    // The kept half of a BlockM x BlockK block of A.  x[] holds Steps * (16 / ES) kept elements per lane.
    template <uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT>
    class __align__(16) fragment<sparse_matrix_a, BlockM, BlockN, BlockK, DataT, row_major>
    {
    public:
        using Shape = detail::SparseShape<BlockM, BlockK, DataT>;
        constexpr static uint32_t num_elements = Shape::Steps * Shape::PerLane;
        using element_type                     = DataT;
        struct Traits
        {
            using StorageT = detail::vec_t<int32_t, Shape::Steps * 4u>;
            constexpr static uint32_t Size = num_elements;
        };
        ROCWMMA_DEVICE fragment() {}
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
            return BlockM;
        }
        ROCWMMA_DEVICE constexpr static inline uint32_t width()
        {
            return BlockK / 2u; // stored elements per row
        }
        ROCWMMA_DEVICE constexpr static inline uint32_t blockDim()
        {
            return BlockM;
        }
        ROCWMMA_DEVICE constexpr static inline uint32_t kDim()
        {
            return BlockK;
        }
        ROCWMMA_DEVICE constexpr static inline uint32_t size()
        {
            return num_elements;
        }
        union
        {
            typename Traits::StorageT mStorage;
            DataT                     x[num_elements];
        };
    };

    // The positions of the kept elements: one index register per instruction.
    template <uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT>
    class __align__(4) fragment<sparse_metadata, BlockM, BlockN, BlockK, DataT, void>
    {
    public:
        using Shape = detail::SparseShape<BlockM, BlockK, DataT>;
        constexpr static uint32_t num_elements = Shape::Steps;
        using element_type                     = uint32_t;
        ROCWMMA_DEVICE fragment() {}
        ROCWMMA_DEVICE inline uint32_t& operator[](uint32_t index)
        {
            return x[index];
        }
        ROCWMMA_DEVICE inline uint32_t const& operator[](uint32_t index) const
        {
            return x[index];
        }
        ROCWMMA_DEVICE constexpr static inline uint32_t size()
        {
            return num_elements;
        }
        uint32_t x[num_elements];
    };

    // values: the block's first byte in the K-blocked storage (Sparse24<DataT>::valueOffset); ldStage: elements
    // between consecutive K stages (Sparse24<DataT>::valueStageStride(m)).  Global or LDS pointers.
    template <uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT>
    ROCWMMA_DEVICE inline void load_matrix_sync(fragment<sparse_matrix_a, BlockM, BlockN, BlockK, DataT, row_major>& frag,
                                                const DataT*                                                         values,
                                                uint32_t                                                             ldStage)
    {
        using Shape         = detail::SparseShape<BlockM, BlockK, DataT>;
        using V             = detail::vec_t<int32_t, 4>;
        const uint32_t lane = threadIdx.x % Constants::AMDGCN_WAVE_SIZE_64;
        const uint32_t row = lane % BlockM, grp = lane / BlockM;
        const char*    base = reinterpret_cast<const char*>(values);
#pragma unroll
        for(uint32_t st = 0; st < Shape::Steps; ++st)
        {
            const uint32_t chunk = st * Shape::G + grp; // 16-byte chunk of the row's kept elements
            const V        v     = *reinterpret_cast<const V*>(base + (uint64_t)(chunk / 4u) * ldStage * Shape::ES
                                                        + Sparse24<DataT>::valueByteInStage(row, chunk % 4u));
            __builtin_memcpy(frag.x + st * Shape::PerLane, &v, 16);
        }
    }

    // meta: the block's first byte of the index storage (Sparse24<DataT>::metaOffset); ldStage: bytes between
    // consecutive K stages (Sparse24<DataT>::metaStageStride(m)).
    template <uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT>
    ROCWMMA_DEVICE inline void load_matrix_sync(fragment<sparse_metadata, BlockM, BlockN, BlockK, DataT, void>& frag,
                                                const uint8_t*                                                  meta,
                                                uint32_t                                                        ldStage)
    {
        using Shape         = detail::SparseShape<BlockM, BlockK, DataT>;
        const uint32_t lane = threadIdx.x % Constants::AMDGCN_WAVE_SIZE_64;
        const uint32_t row = lane % BlockM, grp = lane / BlockM;
#pragma unroll
        for(uint32_t st = 0; st < Shape::Steps; ++st)
        {
            const uint32_t chunk = st * Shape::G + grp;
            const uint8_t* p     = meta + (uint64_t)(chunk / 4u) * ldStage + Sparse24<DataT>::metaByteInStage(row, chunk % 4u);
            if constexpr(Shape::ES == 1u)
                frag.x[st] = *reinterpret_cast<const uint32_t*>(p);
            else
                frag.x[st] = *reinterpret_cast<const uint16_t*>(p);
        }
    }

    // d = A * B + c with A 2:4 sparse; d may alias c.  One v_smfmac_* per StepK of k.
    template <uint32_t BlockM,
              uint32_t BlockN,
              uint32_t BlockK,
              typename InputT,
              typename ComputeT,
              typename LayoutB,
              typename LayoutC,
              typename LayoutD>
    ROCWMMA_DEVICE inline void mma_sync(fragment<accumulator, BlockM, BlockN, BlockK, ComputeT, LayoutD>&           d,
                                        fragment<sparse_matrix_a, BlockM, BlockN, BlockK, InputT, row_major> const& a,
                                        fragment<sparse_metadata, BlockM, BlockN, BlockK, InputT, void> const&      meta,
                                        fragment<matrix_b, BlockM, BlockN, BlockK, InputT, LayoutB> const&          b,
                                        fragment<accumulator, BlockM, BlockN, BlockK, ComputeT, LayoutC> const&     c)
    {
        static_assert(BlockM == BlockN, "sparse mma_sync supports 16x16 and 32x32 blocks");
        using Shape   = detail::SparseShape<BlockM, BlockK, InputT>;
        using LayoutB_ = detail::RegisterLayout<matrix_b, BlockM, BlockN, BlockK, InputT>;
        static_assert(LayoutB_::KW * sizeof(InputT) == 16u && LayoutB_::NumChunks == 2u * Shape::Steps,
                      "matrix_b fragment must hold 16-byte K chunks, two per sparse instruction");
        constexpr bool IsInt = detail::is_i8_v<InputT>;
        using AccE           = std::conditional_t<IsInt, int32_t, float32_t>;
        static_assert(std::is_same_v<ComputeT, AccE>, "sparse accumulators are int32 for int8 and float otherwise");
        constexpr uint32_t AccN = BlockM == 32u ? 16u : 4u;
        using AccT              = detail::vec_t<AccE, AccN>;
        AccT acc;
        __builtin_memcpy(&acc, c.x, sizeof(AccT));
#if ROCWMMA_DEVICE_COMPILE
#pragma unroll
        for(uint32_t st = 0; st < Shape::Steps; ++st)
        {
            const int idx = static_cast<int>(meta.x[st]);
            if constexpr(sizeof(InputT) == 1u)
            {
                detail::vec_t<int, 4> av;
                detail::vec_t<int, 8> bv;
                __builtin_memcpy(&av, a.x + st * 16u, 16);
                __builtin_memcpy(&bv, b.x + st * 32u, 32);
                if constexpr(IsInt && BlockM == 16u)
                    acc = __builtin_amdgcn_smfmac_i32_16x16x128_i8(av, bv, acc, idx, 0, 0);
                else if constexpr(IsInt)
                    acc = __builtin_amdgcn_smfmac_i32_32x32x64_i8(av, bv, acc, idx, 0, 0);
                else if constexpr(detail::is_fp8_v<InputT> && BlockM == 16u)
                    acc = __builtin_amdgcn_smfmac_f32_16x16x128_fp8_fp8(av, bv, acc, idx, 0, 0);
                else if constexpr(detail::is_fp8_v<InputT>)
                    acc = __builtin_amdgcn_smfmac_f32_32x32x64_fp8_fp8(av, bv, acc, idx, 0, 0);
                else if constexpr(BlockM == 16u)
                    acc = __builtin_amdgcn_smfmac_f32_16x16x128_bf8_bf8(av, bv, acc, idx, 0, 0);
                else
                    acc = __builtin_amdgcn_smfmac_f32_32x32x64_bf8_bf8(av, bv, acc, idx, 0, 0);
            }
            else if constexpr(detail::is_f16_v<InputT>)
            {
                detail::vec_t<_Float16, 8>  av;
                detail::vec_t<_Float16, 16> bv;
                __builtin_memcpy(&av, a.x + st * 8u, 16);
                __builtin_memcpy(&bv, b.x + st * 16u, 32);
                if constexpr(BlockM == 16u)
                    acc = __builtin_amdgcn_smfmac_f32_16x16x64_f16(av, bv, acc, idx, 0, 0);
                else
                    acc = __builtin_amdgcn_smfmac_f32_32x32x32_f16(av, bv, acc, idx, 0, 0);
            }
            else
            {
                static_assert(detail::is_bf16_v<InputT>, "sparse matrix instructions: int8, fp8, bf8, f16, bf16");
                detail::vec_t<__bf16, 8>  av;
                detail::vec_t<__bf16, 16> bv;
                __builtin_memcpy(&av, a.x + st * 8u, 16);
                __builtin_memcpy(&bv, b.x + st * 16u, 32);
                if constexpr(BlockM == 16u)
                    acc = __builtin_amdgcn_smfmac_f32_16x16x64_bf16(av, bv, acc, idx, 0, 0);
                else
                    acc = __builtin_amdgcn_smfmac_f32_32x32x32_bf16(av, bv, acc, idx, 0, 0);
            }
        }
#else
        (void)a;
        (void)meta;
        (void)b;
#endif
        __builtin_memcpy(d.x, &acc, sizeof(AccT));
    }
} // namespace rocwmma

#endif // ROCWMMA_SPARSE_API_HPP
