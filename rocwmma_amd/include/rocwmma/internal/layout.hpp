// Register layouts of fragments and 1-d memory maps.
//
// The reference derives fragment register layouts from a generic stride-space engine
// whose result depends on the memory orientation (layout.hpp:120-269,
// layout_impl.hpp:98-617, io_layout.hpp:38-207).  Here a fragment's register layout
// is fixed by the gfx950 MFMA operand format and depends only on
// (matrix role, block shape, data type) -- never on the memory orientation -- so that
// applyTranspose / applyDataLayout and the runtime-layout load/store overloads are
// pure reinterpretations.
//
// One formula covers A, B and accumulator fragments.  Let BlockDim be the non-reduced
// dimension held across lanes and KDim the other one (io_shape.hpp:43-80):
//     D  = min(BlockDim, 64)      lanes spanning BlockDim
//     G  = 64 / D                 lane groups spanning KDim
//     KW                          consecutive KDim elements one lane holds per chunk
// lane l, element e of a fragment (E = KDim / G elements per BlockDim segment):
//     seg = e / E,  r = e % E
//     dim = seg * D + l % D
//     k   = (r / KW) * (KW * G) + (l / D) * KW + r % KW
// For BlockDim 16 / 32 a chunk of KW * G along K is exactly one MFMA operand:
//   f16, bf16 : KW 8 -> v_mfma_f32_32x32x16 / 16x16x32,  KW 4 -> 32x32x8 / 16x16x16
//   int8      : KW 16 -> v_mfma_i32_32x32x32 / 16x16x64, KW 8 -> 32x32x16 / 16x16x32
//   fp8 / bf8 : KW 16 -> two v_mfma_f32_32x32x16 / 16x16x32 (fp8_fp8 / bf8_bf8) on the lane's two 8-byte halves,
//               KW 8 -> one (a lane's 16 consecutive K bytes are also what the 2:4 sparse instructions pair with)
//   f32       : KW 1 -> v_mfma_f32_32x32x2 / 16x16x4
//   f64       : KW 1 -> v_mfma_f64_16x16x4 (BlockDim 16 only)
// Accumulators use KW 4, which is the MFMA C/D layout (f64: KW 1, row = 4 e + lane / 16)
//   (32x32: col = l % 32, row = 8 * (e / 4) + 4 * (l / 32) + e % 4;
//    16x16: col = l % 16, row = 4 * (l / 16) + e)
// for every element type, so `fragC.x[i]` and `fragAcc.x[i]` always name the same (row, col).
//
// Staging fragments (matrix_a / matrix_b with BlockDim >= 64: the macro-tile buffers of cooperative kernels,
// which are only loaded and stored, never multiplied) hold vectors along BlockDim instead: a chunk is V = 16 bytes'
// worth of consecutive BlockDim elements at one k,
//     BlockDim / V >= 64 :  chunk c, lane l:  k = c / P,  dim = V * (64 * (c % P) + l),   P = BlockDim / V / 64
//     BlockDim / V <  64 :  chunk c, lane l:  k = c * R + l / (BlockDim / V),  dim = V * (l % (BlockDim / V)),
//                           R = 64 V / BlockDim k-rows per chunk
// so that global -> register -> LDS moves of an operand whose BlockDim is the contiguous memory dimension (A
// col-major, B row-major: the orientation of the reference's perf samples) are 128-bit accesses, and the matrix
// fragments then come out of such an LDS image with transposing reads (io.hpp).  Like every other layout here it
// does not depend on the memory orientation: the transforms stay relabels.
#ifndef ROCWMMA_LAYOUT_HPP
#define ROCWMMA_LAYOUT_HPP

#include "constants.hpp"
#include "types.hpp"
#include "utils.hpp"

namespace rocwmma
{
    namespace detail
    {
        // 1-d offset of a (row, col) coordinate; the public face is GetDataLayout_t<Frag>.
        // Reference: mapping_util.hpp:90-107, mapping_util_impl.hpp:142-149.
        template <typename DataOrientation>
        struct DataSpace
        {
            using MatrixCoordT = Coord2d;
            using MatrixSizeT  = Coord2d;
            using Orientation  = DataOrientation;

            enum : uint32_t
            {
                MajorIndex = std::is_same_v<DataOrientation, row_major> ? 0u : 1u,
                MinorIndex = std::is_same_v<DataOrientation, row_major> ? 1u : 0u
            };

            // Size of the contiguous dimension of a (rows, cols) matrix
            ROCWMMA_HOST_DEVICE constexpr static inline uint32_t
                leadingDim(MatrixSizeT const& matrixSize)
            {
                return get<MinorIndex>(matrixSize);
            }

            ROCWMMA_HOST_DEVICE constexpr static inline uint32_t
                fromMatrixCoord(MatrixCoordT const& matrixCoord, uint32_t leadingDim)
            {
                return get<MajorIndex>(matrixCoord) * leadingDim + get<MinorIndex>(matrixCoord);
            }
        };

        template <>
        struct DataSpace<void>
        {
            using MatrixCoordT = Coord2d;
            using MatrixSizeT  = Coord2d;
            using Orientation  = void;
        };

        // Candidate K-widths per lane, widest first, for input (A / B) fragments.
        template <typename DataT>
        constexpr inline uint32_t inputKW(uint32_t kDim, uint32_t groups, bool mfmaShape)
        {
            constexpr uint32_t bytes = sizeof(DataT);
            if(!mfmaShape)
            {
                // cooperative / staging fragments: widest 16-byte vector that tiles KDim
                uint32_t kw = 16u / bytes;
                while(kw > 1u && (kDim % (kw * groups)) != 0u)
                    kw >>= 1;
                return kw;
            }
            // 16 x 16 and 32 x 32 blocks: start from the widest matrix-instruction operand of the type and
            // halve until the wave's chunk tiles KDim.  Widths below the narrowest instruction form (4 for
            // 16-bit types, 8 for 8-bit types) still load, store and fill; mma_sync rejects them.
            uint32_t kw = bytes == 2u ? 8u : (bytes == 1u ? 16u : 1u);
            while(kw > 1u && (kDim % (kw * groups)) != 0u)
                kw >>= 1;
            return kw;
        }

        // Vector length along BlockDim of a staging fragment; 0: the fragment holds vectors along K
        template <typename DataT>
        constexpr inline uint32_t dimVector(uint32_t blockDim, uint32_t kDim, bool input)
        {
            if(!input || blockDim < 64u)
                return 0u;
            for(uint32_t v = 16u / static_cast<uint32_t>(sizeof(DataT)); v > 1u; v >>= 1)
            {
                if(blockDim % v)
                    continue;
                const uint32_t lanesPerRow = blockDim / v;
                if(lanesPerRow >= 64u ? lanesPerRow % 64u == 0u : (64u % lanesPerRow == 0u && kDim % (64u / lanesPerRow) == 0u))
                    return v;
            }
            return 0u;
        }

        template <typename MatrixT, uint32_t BlockM, uint32_t BlockN, uint32_t BlockK, typename DataT>
        struct RegisterLayout
        {
            static constexpr bool IsA   = std::is_same_v<MatrixT, matrix_a>;
            static constexpr bool IsB   = std::is_same_v<MatrixT, matrix_b>;
            static constexpr bool IsAcc = std::is_same_v<MatrixT, accumulator>;
            static_assert(IsA || IsB || IsAcc, "MatrixT must be matrix_a, matrix_b or accumulator");

            static constexpr uint32_t WaveSize    = Constants::AMDGCN_WAVE_SIZE_64;
            static constexpr uint32_t BlockHeight = IsA ? BlockM : (IsB ? BlockK : BlockM);
            static constexpr uint32_t BlockWidth  = IsA ? BlockK : (IsB ? BlockN : BlockN);
            static constexpr uint32_t BlockDim    = IsA ? BlockM : BlockN;
            static constexpr uint32_t KDim        = IsAcc ? BlockM : BlockK;

            static_assert(isPow2(BlockDim), "BlockDim must be a power of two");

            static constexpr uint32_t D    = cmin(BlockDim, WaveSize);
            static constexpr uint32_t G    = WaveSize / D;
            static constexpr uint32_t Segs = BlockDim / D;
            // staging fragments: vectors of DimV consecutive BlockDim elements
            static constexpr uint32_t DimV        = dimVector<DataT>(BlockDim, KDim, !IsAcc);
            static constexpr bool     VecAlongDim = DimV != 0u;
            static constexpr uint32_t LanesPerRow = VecAlongDim ? BlockDim / DimV : 1u;
            static constexpr uint32_t PassesPerRow = LanesPerRow >= WaveSize ? LanesPerRow / WaveSize : 1u;
            static constexpr uint32_t RowsPerPass  = LanesPerRow >= WaveSize ? 1u : WaveSize / LanesPerRow;
            // elements per chunk: along K (f64 accumulators follow v_mfma_f64_16x16x4: one row per register, rows G
            // apart), or along BlockDim for staging fragments
            static constexpr uint32_t KW
                = VecAlongDim ? DimV
                              : (IsAcc ? (sizeof(DataT) == 8u ? 1u : 4u)
                                       : inputKW<DataT>(KDim, G, BlockDim == 16u || BlockDim == 32u));

            static_assert(VecAlongDim || KDim % (KW * G) == 0u,
                          "KDim is not a multiple of the K extent one wave holds per register chunk");

            static constexpr uint32_t ElementsPerSeg = KDim / G;
            static constexpr uint32_t ChunksPerSeg   = VecAlongDim ? 1u : ElementsPerSeg / KW;
            static constexpr uint32_t NumElements    = Segs * ElementsPerSeg;
            static constexpr uint32_t NumChunks      = NumElements / KW;
            static constexpr uint32_t ChunkK         = VecAlongDim ? RowsPerPass : KW * G; // K extent of one chunk over the wave

            static_assert(NumElements * sizeof(DataT) >= 4u && (NumElements * sizeof(DataT)) % 4u == 0u,
                          "Fragments must occupy at least one packed register");

            // (BlockDim index, KDim index) of the first element of chunk c for lane l
            ROCWMMA_DEVICE static inline uint32_t dimOf(uint32_t lane, uint32_t chunk)
            {
                if constexpr(VecAlongDim)
                    return DimV * (LanesPerRow >= WaveSize ? WaveSize * (chunk % PassesPerRow) + lane : lane % LanesPerRow);
                else
                    return (chunk / ChunksPerSeg) * D + lane % D;
            }
            ROCWMMA_DEVICE static inline uint32_t kOf(uint32_t lane, uint32_t chunk)
            {
                if constexpr(VecAlongDim)
                    return LanesPerRow >= WaveSize ? chunk / PassesPerRow : chunk * RowsPerPass + lane / LanesPerRow;
                else
                    return (chunk % ChunksPerSeg) * ChunkK + (lane / D) * KW;
            }
            // (row, col) of BlockDim index d and KDim index k
            ROCWMMA_HOST_DEVICE constexpr static inline Coord2d matrixCoord(uint32_t d, uint32_t k)
            {
                return IsA ? Coord2d{d, k} : Coord2d{k, d};
            }
        };

        // True when consecutive KDim elements are consecutive in memory
        template <typename MatrixT, typename DataLayoutT>
        inline constexpr bool kContiguous_v
            = std::is_same_v<MatrixT, matrix_a> ? std::is_same_v<DataLayoutT, row_major>
                                                : std::is_same_v<DataLayoutT, col_major>;
    } // namespace detail
    // Public names of the 1-d data spaces (reference: layout/data_layout.hpp, used by kernels as
    // DataLayout::Array1d<row_major>::fromMatrixCoord(coord, ld)).
    namespace DataLayout
    {
        template <typename DataOrientation>
        using Array1d = detail::DataSpace<DataOrientation>;
        using RowMajor = Array1d<row_major>;
        using ColMajor = Array1d<col_major>;
    } // namespace DataLayout

} // namespace rocwmma

#endif // ROCWMMA_LAYOUT_HPP
