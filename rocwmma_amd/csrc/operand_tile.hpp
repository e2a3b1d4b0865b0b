// Operand tiles of the macro-tile kernels in LDS: where a lane's 16-byte chunk of a K stage lies in global memory and in
// LDS, and how a wave reads its operand blocks back.  Shared by the dense kernels (gemm_tiled.hip) and the 2:4 sparse one
// (sparse.hip, dense B).
//
// A stage is 128 bytes of K.  An operand tile of 32 WB rows (WB = 8: 256 rows, 32 KiB; WB = 4: 128 rows, 16 KiB) is
// written by direct loads, chunk L = j * 256 + tid at LDS byte 16 L:
//   * K-contiguous (A row-major / B col-major): rows x 128 B, chunk c of row r in slot c ^ ((r >> 1) & 7); a lane
//     reads 16 consecutive K bytes of its row with one ds_read_b128;
//   * M/N-contiguous (A col-major / B row-major): k-rows x (32 WB ES) B with a swizzle that depends on the element
//     size (swzMN8); 1- and 2-byte elements come back through transposing reads (ds_read_b64_tr_b8 / _b16), two per
//     16-byte piece of an operand block.
#ifndef R355_OPERAND_TILE_HPP
#define R355_OPERAND_TILE_HPP

#include <cstdint>

#include <hip/hip_runtime.h>

namespace r355
{
    namespace tile
    {
        constexpr uint32_t STAGE_KB = 128; // bytes of K per stage per row
        constexpr uint32_t THREADS  = 256;
        constexpr uint32_t CHUNK    = 16; // bytes moved per lane per access
        using i32x4  = int __attribute__((ext_vector_type(4)));
        using i32x2  = int __attribute__((ext_vector_type(2)));
        typedef __fp16 trv4 __attribute__((__vector_size__(4 * sizeof(__fp16)))); // operand type of the transposing LDS read

        __device__ __forceinline__ uint32_t swzK8(uint32_t row)
        {
            return (row >> 1) & 7u;
        }
        template <uint32_t WB, uint32_t ES = 1>
        __device__ __forceinline__ uint32_t swzMN8(uint32_t krow)
        {
            if constexpr(ES == 8)
                return ((krow >> 1) & 1u) << 3; // f64: a 32-lane pass reads two k-rows 2 apart, 128 bytes each
            else if constexpr(ES == 4)
                return ((krow >> 2) & 3u) << 2; // f32: a wave reads k-rows 4 apart, 64 bytes each
            else if constexpr(ES == 2)
                return ((krow & 3u) << 2) | (((krow >> 3) & 1u) << 1); // 16-bit elements: as in gemmTiled16
            else if constexpr(WB == 8)
                return (krow & 7u) | ((krow >> 1) & 8u); // 256-byte k-rows, 16 chunks
            else
                return ((krow >> 1) & 3u) | ((krow >> 2) & 4u); // 128-byte k-rows, 8 chunks: rows 2 apart share banks
        }

        // global -> LDS lane offsets of one operand: load j brings chunk j * 256 + tid.  Edge tiles (m or
        // n not a multiple of 256) must not read outside the operand: a lane whose row (K-contiguous) or
        // chunk (M/N-contiguous) lies beyond the matrix reads the last valid row / the first chunk instead;
        // what lands in LDS for it only feeds elements of D that are never stored.  `step` is the uniform
        // offset from one load to the next, `stage` the distance between K stages, `kByte` the K offset
        // inside a stage of a K-contiguous lane's chunks.
        // (ES = element size in bytes: the five-buffer kernel body below also serves 16-bit operands, whose
        // M/N-contiguous tiles are 64 k-rows of 64 WB bytes read with ds_read_b64_tr_b16)
        template <bool KCONTIG, uint32_t WB, uint32_t ES = 1>
        __device__ __forceinline__ void laneOffsets8(uint32_t tid, uint32_t ld, uint32_t valid, uint32_t (&off)[WB], uint32_t& step,
                                                     uint64_t& stage, uint32_t& kByte)
        {
            kByte = 0u;
            if constexpr(KCONTIG)
            {
                const uint32_t r = tid >> 3, slot = tid & 7u; // row 32 j + r
                kByte = (slot ^ swzK8(r)) * CHUNK;
    #pragma unroll
                for(uint32_t j = 0; j < WB; ++j)
                {
                    const uint32_t row = r + 32u * j < valid ? r + 32u * j : valid - 1u;
                    off[j]             = row * ld * ES + ((slot ^ swzK8(r)) * CHUNK);
                }
                step = 0u, stage = STAGE_KB;
            }
            else
            {
                constexpr uint32_t SLOTS = 2u * WB * ES, KROWS = THREADS / SLOTS; // chunks per k-row, k-rows per load
                const uint32_t     r = tid / SLOTS, slot = tid % SLOTS; // k-row KROWS j + r (the swizzle may alternate with j)
    #pragma unroll
                for(uint32_t j = 0; j < WB; ++j)
                {
                    const uint32_t c = slot ^ swzMN8<WB, ES>(KROWS * j + r);
                    off[j]           = r * ld * ES + (c * (CHUNK / ES) < valid ? c : 0u) * CHUNK;
                }
                step = KROWS * ld * ES, stage = (uint64_t)STAGE_KB * ld;
            }
        }

        // LDS -> register lane offsets of one operand for the wave whose tile starts at row 16 WB w.
        // K-contiguous: rd[q] is 64-byte K step q of block 0 (block i is 16 rows further);
        // M/N-contiguous: rd[i] is block i, the first 8 k-rows of the lane's 16 of K step 0.
        template <bool KCONTIG, uint32_t WB, uint32_t ES = 1>
        __device__ __forceinline__ void readOffsets8(uint32_t w, uint32_t lane, uint32_t (&rd)[8])
        {
            const uint32_t t = lane & 15u, g = lane >> 4;
    #pragma unroll
            for(uint32_t i = 0; i < 8; ++i)
                rd[i] = 0u;
            if constexpr(KCONTIG)
            {
                const uint32_t r = w * 16u * WB + t;
                rd[0]            = r * STAGE_KB + ((g ^ swzK8(r)) * CHUNK);
                rd[1]            = r * STAGE_KB + (((4u + g) ^ swzK8(r)) * CHUNK);
            }
            else if constexpr(ES == 1)
            {
                const uint32_t kr = 16u * g + (t >> 1);
    #pragma unroll
                for(uint32_t i = 0; i < WB; ++i)
                    rd[i] = kr * 32u * WB + (((w * WB + i) ^ swzMN8<WB>(kr)) * CHUNK) + (t & 1u) * 8u;
            }
            else if constexpr(ES == 8)
            {
                // f64: element e of the lane's two K values is k-row 2 (lane / 16) + e of the K step, column lane % 16
                const uint32_t kr = 2u * g;
    #pragma unroll
                for(uint32_t i = 0; i < WB; ++i)
                    rd[i] = kr * 256u * WB + ((((w * 8u * WB + 8u * i) ^ swzMN8<WB, 8>(kr)) + (t >> 1)) * CHUNK) + (t & 1u) * 8u;
            }
            else if constexpr(ES == 4)
            {
                // f32 (no transposing read for 32-bit elements): element e of the lane's four K values is k-row
                // 4 (lane / 16) + e of the K step, column lane % 16 of the block -- 64 consecutive bytes per 16 lanes
                const uint32_t kr = 4u * g;
    #pragma unroll
                for(uint32_t i = 0; i < WB; ++i)
                    rd[i] = kr * 128u * WB + ((((w * 4u * WB + 4u * i) ^ swzMN8<WB, 4>(kr)) + (t >> 2)) * CHUNK) + (t & 3u) * 4u;
            }
            else
            {
                // 16-bit: k-row 8 (lane / 16) + (lane % 16) / 4 of the K step's first half, 8-byte piece 4 i + lane % 4
                const uint32_t kr = 8u * g + (t >> 2);
    #pragma unroll
                for(uint32_t i = 0; i < WB; ++i)
                {
                    const uint32_t piece = w * 4u * WB + 4u * i + (t & 3u);
                    rd[i] = kr * 64u * WB + (((piece >> 1) ^ swzMN8<WB, 2>(kr)) * CHUNK) + (piece & 1u) * 8u;
                }
            }
        }

        // 16 K bytes of block i, K step s (64 bytes), of the operand tile at `tile`: they arrive whole with
        // part 0 (K-contiguous) or as two transposed halves, parts 0 and 1, into registers at, at + 1 and
        // at + 2, at + 3 of `dst`
        template <bool KCONTIG, uint32_t WB, uint32_t ES = 1, typename V>
        __device__ __forceinline__ void readBlock8(const char* tile, const uint32_t (&rd)[8], uint32_t i, uint32_t s, uint32_t part,
                                                   V& dst, uint32_t at)
        {
            if constexpr(KCONTIG)
            {
                if(part == 0u)
                {
                    const i32x4 v = *reinterpret_cast<const i32x4*>(tile + rd[s] + i * 16u * STAGE_KB);
                    dst[at] = v[0], dst[at + 1u] = v[1], dst[at + 2u] = v[2], dst[at + 3u] = v[3];
                }
            }
            else if constexpr(ES == 1)
            {
                using lp      = __attribute__((address_space(3))) i32x2*;
                const i32x2 v = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lp)(tile + rd[i] + (64u * s + 8u * part) * 32u * WB));
                dst[at + 2u * part] = v[0], dst[at + 2u * part + 1u] = v[1];
            }
            else if constexpr(ES == 8)
            {
                const i32x2 v = *reinterpret_cast<const i32x2*>(tile + rd[i] + (8u * s + part) * 256u * WB);
                dst[at + 2u * part] = v[0], dst[at + 2u * part + 1u] = v[1];
            }
            else if constexpr(ES == 4)
            {
                const char* q = tile + rd[i] + (16u * s + 2u * part) * 128u * WB;
                dst[at + 2u * part]      = *reinterpret_cast<const int*>(q);
                dst[at + 2u * part + 1u] = *reinterpret_cast<const int*>(q + 128u * WB);
            }
            else
            {
                using lp      = __attribute__((address_space(3))) trv4*;
                const i32x2 v = __builtin_bit_cast(
                    i32x2, __builtin_amdgcn_ds_read_tr16_b64_v4f16((lp)(tile + rd[i] + (32u * s + 4u * part) * 64u * WB)));
                dst[at + 2u * part] = v[0], dst[at + 2u * part + 1u] = v[1];
            }
        }

    } // namespace tile
} // namespace r355

#endif // R355_OPERAND_TILE_HPP
