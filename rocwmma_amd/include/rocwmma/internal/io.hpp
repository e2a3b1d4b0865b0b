// Fragment <-> memory movement for one wave (and for a share of a cooperative fragment).
//
// Reference counterparts: opaque_load.hpp:59-140, opaque_store.hpp:57-134 (whole
// fragment per wave) and coop_load.hpp:107-218, coop_store.hpp:108-222 (stride space
// split over waves).  Here a fragment is a list of register chunks (KW consecutive
// elements each -- along KDim, or along BlockDim for staging fragments, see layout.hpp); a
// chunk moves as one vector access when its direction is the contiguous memory dimension
// and as KW element accesses, coalesced across lanes, otherwise.  One exception: a matrix
// fragment (16 or 32 rows / columns, 8- or 16-bit elements) whose BlockDim is the contiguous
// dimension of an LDS image is fetched with the transposing LDS reads of gfx950
// (ds_read_b64_tr_b16 / _b8: 16 lanes name a 4 x 16 or 8 x 16 element block and each receives one
// column of it), one or two reads per chunk instead of KW element reads.  Pointers may be
// global or LDS; vector accesses need the natural alignment of KW elements, as the
// reference's vector-width accesses do.
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

            static constexpr uint32_t KW = Layout::KW;
            // the bits of one chunk as a naturally aligned vector
            static constexpr uint32_t ChunkBytes = KW * sizeof(DataT);
            using Bits = std::conditional_t<
                ChunkBytes % 4u == 0u,
                vec_t<uint32_t, (ChunkBytes >= 4u ? ChunkBytes / 4u : 1u)>,
                std::conditional_t<ChunkBytes == 2u, uint16_t, std::conditional_t<ChunkBytes == 1u, uint8_t, Packet<DataT, KW>>>>;
            static_assert(sizeof(Bits) == ChunkBytes, "chunk vector must cover the chunk exactly");
            // a chunk runs along K (matrix fragments) or along BlockDim (staging fragments)
            static constexpr bool Contiguous
                = Layout::VecAlongDim ? !kContiguous_v<MatrixT, DataLayoutT> : kContiguous_v<MatrixT, DataLayoutT>;
            // transposing LDS reads: K-major registers out of a BlockDim-contiguous image
            static constexpr uint32_t TrK = sizeof(DataT) == 2u ? 4u : 8u; // K elements one transposing read delivers
            static constexpr bool     TrCapable
                = !Contiguous && !Layout::VecAlongDim && !Layout::IsAcc && (Layout::BlockDim == 16u || Layout::BlockDim == 32u)
                  && (sizeof(DataT) == 1u || sizeof(DataT) == 2u) && KW % TrK == 0u;

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

            // Elements of 8 or 16 bits that arrived one by one sit in a 32-bit register each for as long as the compiler
            // sees them as separate values: the 64 halves of four 32 x 32 accumulator blocks loaded ahead of an epilogue
            // then hold 64 registers.  Passing every 32-bit word of the chunk through an opaque statement makes the packed
            // word the value that stays live (one v_perm / v_lshl_or per word; unpacking at the use is an operand select).
            ROCWMMA_DEVICE static inline void keepPacked(DataT* chunk)
            {
#if ROCWMMA_DEVICE_COMPILE
                if constexpr(Layout::IsAcc && sizeof(DataT) < 4u && ChunkBytes % 4u == 0u)
                {
#pragma unroll
                    for(uint32_t w = 0; w < ChunkBytes / 4u; ++w)
                    {
                        uint32_t word;
                        __builtin_memcpy(&word, reinterpret_cast<char*>(chunk) + 4u * w, 4);
                        asm volatile("" : "+v"(word));
                        __builtin_memcpy(reinterpret_cast<char*>(chunk) + 4u * w, &word, 4);
                    }
                }
#else
                (void)chunk;
#endif
            }

            // An offset (or leading dimension) the compiler cannot use before this point of the program, for the
            // element accesses of accumulator fragments: the addresses of a block's 16 or 64 accesses, and the offsets
            // they share with the next block's, are otherwise all formed ahead and held in registers, and that
            // footprint sets the occupancy of a kernel whose epilogue uses these accesses (the reference's perf_hgemm
            // sample through these headers: 132 -> 101 registers, 2 -> 3 waves per SIMD, 274 -> 364 TFLOP/s).  Matrix
            // fragments keep free scheduling: their element loads sit in K loops, where ordering them costs more
            // than the registers.
            ROCWMMA_DEVICE static inline uint32_t justInTime(uint32_t off)
            {
#if ROCWMMA_DEVICE_COMPILE
                if constexpr(Layout::IsAcc)
                    asm volatile("" : "+v"(off) : : "memory");
#endif
                return off;
            }

            // Chunks [FirstChunk, FirstChunk + Count) of memory <-> registers [RegChunk...)
            template <uint32_t Count>
            ROCWMMA_DEVICE static inline void
                load(DataT* regs, DataT const* data, uint32_t ldm, uint32_t firstChunk)
            {
                const uint32_t l = lane();
#if ROCWMMA_DEVICE_COMPILE && !defined(ROCWMMA_NO_TR_READS)
                if constexpr(TrCapable)
                {
                    // 8-byte pieces: the image's rows (ldm) and base must keep them aligned.  The test is made a scalar
                    // (the block address is the same for the whole wave) so that the other path is branched over, never
                    // run with an empty execution mask: a transposing read exchanges data between lanes and is meant
                    // for full waves only.
                    const bool inLds = __builtin_amdgcn_is_shared(static_cast<const void*>(data))
                                       && (ldm * sizeof(DataT)) % 8u == 0u && reinterpret_cast<unsigned long long>(data) % 8u == 0u;
                    if(__builtin_amdgcn_readfirstlane(static_cast<int>(inLds)) != 0)
                    {
                        // lane t of each group of 16 names the piece at k-row t / (16 / TrK), BlockDim offset
                        // (8 / sizeof) * (t % (16 / TrK)) of the group's TrK x 16 block and receives the TrK k values
                        // of its own row / column l % 16
                        constexpr uint32_t PiecesPerRow = 16u / TrK; // 8-byte pieces per k-row of the block: 4 or 2
                        const uint32_t     t = l % 16u;
#pragma unroll
                        for(uint32_t c = 0; c < Count; ++c)
                        {
                            const uint32_t d0 = Layout::dimOf(l, firstChunk + c) - t; // the 16-lane group's first row / column
                            const uint32_t k0 = Layout::kOf(l, firstChunk + c);
#pragma unroll
                            for(uint32_t h = 0; h < KW / TrK; ++h)
                            {
                                const DataT* src = data + offset(d0 + (8u / sizeof(DataT)) * (t % PiecesPerRow), k0 + TrK * h + t / PiecesPerRow, ldm);
                                if constexpr(sizeof(DataT) == 2u)
                                {
                                    using V4 = short __attribute__((ext_vector_type(4)));
                                    const V4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                                        (__attribute__((address_space(3))) V4*)(const_cast<V4*>(reinterpret_cast<const V4*>(src))));
                                    __builtin_memcpy(regs + c * KW + TrK * h, &v, 8);
                                }
                                else
                                {
                                    using V2 = int __attribute__((ext_vector_type(2)));
                                    const V2 v = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
                                        (__attribute__((address_space(3))) V2*)(const_cast<V2*>(reinterpret_cast<const V2*>(src))));
                                    __builtin_memcpy(regs + c * KW + TrK * h, &v, 8);
                                }
                            }
                        }
                        return;
                    }
                }
#endif
#pragma unroll
                for(uint32_t c = 0; c < Count; ++c)
                {
                    const uint32_t d = Layout::dimOf(l, firstChunk + c);
                    const uint32_t k = Layout::kOf(l, firstChunk + c);
                    if constexpr(Contiguous)
                    {
                        // one vector access; the registers are written through a copy of known size (a vector store
                        // through a cast pointer into the fragment keeps the compiler from splitting the fragment
                        // into registers: it then lives in scratch memory)
                        const Bits v = *reinterpret_cast<Bits const*>(data + offset(d, k, ldm));
                        __builtin_memcpy(regs + c * KW, &v, sizeof(Bits));
                    }
                    else
                    {
                        const uint32_t ld   = justInTime(ldm);
                        const uint32_t base = offset(d, k, ld);
#pragma unroll
                        for(uint32_t e = 0; e < KW; ++e)
                            regs[c * KW + e] = data[justInTime(base + e * ld)];
                    }
                }
                // (after the last access has been issued: the statement waits for the data it is given)
                if constexpr(!Contiguous)
                {
#pragma unroll
                    for(uint32_t c = 0; c < Count; ++c)
                        keepPacked(regs + c * KW);
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
                        Bits v;
                        __builtin_memcpy(&v, regs + c * KW, sizeof(Bits));
                        *reinterpret_cast<Bits*>(data + offset(d, k, ldm)) = v;
                    }
                    else
                    {
                        const uint32_t ld   = justInTime(ldm);
                        const uint32_t base = offset(d, k, ld);
#pragma unroll
                        for(uint32_t e = 0; e < KW; ++e)
                            data[justInTime(base + e * ld)] = regs[c * KW + e];
                    }
                }
            }
        };
    } // namespace detail
} // namespace rocwmma

#endif // ROCWMMA_IO_HPP
