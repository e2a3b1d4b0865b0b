// LDS-staged macro-tile GEMM for gfx950, written directly against the hardware (no fragment-API
// composition).
//
// Takes the place of samples/perf_hgemm.cpp:515-711 and
// test/gemm/gemm_PGR1_LB2_MP0_MB_CP/device/kernel_device_func.hpp:52-283.  The reference
// kernel moves 128x128x16 macro tiles through 16 KiB of LDS with element-wise LDS reads
// and eight matrix instructions per wave between barriers; this one is shaped for
// MI355X's 160 KB LDS and 256 CUs:
//
//   macro tile   256 x 256, K stage of 128 bytes (64 f16/bf16, 128 int8/fp8 elements); 128 x 128 (wave tile
//                64 x 64, five 16 KiB LDS buffers, two workgroups per CU) for problems with too few large tiles
//   workgroup    256 threads = 4 waves in a 2 x 2 grid, wave tile 128 x 128
//                = 8 x 8 accumulators of the 16 x 16 matrix-instruction shapes (256 registers):
//                v_mfma_f32_16x16x32_{f16,bf16}, v_mfma_i32_16x16x64_i8, v_mfma_f32_16x16x128_f8f6f4.
//                Under the board's power limit these sustain 12-20 % more than the 32 x 32 shapes of
//                the same types (register-resident loops, random operands), and the kernels are
//                power-bound.
//   LDS          16-bit types: 2 stages x (A 32 KiB + B 32 KiB) = 128 KiB;
//                8-bit types: 2 A buffers + 3 B buffers x 32 KiB = 160 KiB;
//                one workgroup per CU either way
//   global->LDS  128-bit loads written straight into LDS by the memory pipeline
//                (buffer_load_dwordx4 ... lds), no register staging
//   LDS layout   16-byte chunks, XOR-swizzled inside each row so that both the
//                row-contiguous writes and the MFMA-shaped reads are bank-conflict free
//   LDS->regs    K-contiguous operands: one ds_read_b128 per 16-row operand block;
//                M/N-contiguous operands: two ds_read_b64_tr_b16 / ds_read_b64_tr_b8 (transposing
//                reads) -- no element-wise reads anywhere; operands are fetched one K step
//                (64 matrix instructions; fp8: one quadrant, 16) ahead of their use
//   schedule     the matrix instructions are inline assembly with the accumulator tied in place
//                (the compiler's own selection leaves the 64 small accumulators untied and its
//                register allocator then shuffles them through the K loop), so the kernels fix
//                the instruction order themselves: one LDS read or direct load per matrix
//                instruction, pinned by scheduling barriers
//   shapes       m, n multiples of 16 and k a multiple of a 16-byte chunk: edge tiles clamp their loads and guard
//                their stores, a partial last K stage is completed with zeros by out-of-range buffer loads
//   grid         1-D, remapped so that each XCD (workgroup id mod 8) owns a compact
//                rectangle of tiles and walks it in 4-row groups (L2 reuse of A and B)
//
// Operand orientation is a template parameter per operand ("K-contiguous" = A row-major /
// B col-major).  The MFMA operands are swapped so that each lane holds four consecutive
// columns of a row of D; a col-major D is computed as the row-major D^T = B^T A^T.
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <type_traits>

#include "common.hpp"
#include "lds_dma.hpp"
#include "operand_tile.hpp"
#include "tile_map.hpp"

// This file is compiled once per part so that its kernel families build in parallel: part 0 holds the host
// side and the f16 kernels, part 1 bf16, part 2 the 8-bit types, part 3 f32 and f64.  Without the macro one
// translation unit holds everything.
#ifndef R355_TILED_PART
#define R355_TILED_PART (-1)
#endif
#define R355_TILED_HAS(part) (R355_TILED_PART < 0 || R355_TILED_PART == (part))

// Profiling build (-DR355_TIMELINE, `python -m rocwmma_amd.build --timeline`; never the shipped library): thread 0 of every
// workgroup of the 256 x 256 tile kernels records the 100 MHz counter at entry (0), when the first stage is in LDS (1),
// after the K loop (2) and after the last store has been issued and acknowledged (3), and its hardware id (4, 5).
// `python -m rocwmma_amd.timeline` reads the records through r355_timeline_read_p<part>.
#ifdef R355_TIMELINE
#define R355_TL_PASTE2(a, b) a##b
#define R355_TL_PASTE(a, b) R355_TL_PASTE2(a, b)
static __device__ unsigned long long r355_timeline[8192 * 8];
extern "C" int R355_TL_PASTE(r355_timeline_read_p, R355_TILED_PART)(void* host, size_t bytes)
{
    return static_cast<int>(hipMemcpyFromSymbol(host, HIP_SYMBOL(r355_timeline), bytes));
}
#define R355_STAMP(slot)                                                                            \
    do                                                                                              \
    {                                                                                               \
        if(WB == 8 && threadIdx.x == 0 && blockIdx.x < 8192u)                                       \
            r355_timeline[blockIdx.x * 8u + (slot)] = __builtin_amdgcn_s_memrealtime();             \
    } while(0)
#define R355_STAMP_ID()                                                                             \
    do                                                                                              \
    {                                                                                               \
        if(WB == 8 && threadIdx.x == 0 && blockIdx.x < 8192u)                                       \
        {                                                                                           \
            r355_timeline[blockIdx.x * 8u + 4u] = __builtin_amdgcn_s_getreg(63492); /* HW_ID */     \
            r355_timeline[blockIdx.x * 8u + 5u] = __builtin_amdgcn_s_getreg(63508); /* XCC_ID */    \
        }                                                                                           \
    } while(0)
#define R355_STAMP_END()                                                                            \
    do                                                                                              \
    {                                                                                               \
        __builtin_amdgcn_s_waitcnt(0);                                                              \
        R355_STAMP(3);                                                                              \
    } while(0)
#else
#define R355_STAMP(slot)
#define R355_STAMP_ID()
#define R355_STAMP_END()
#endif

namespace r355
{
    struct GemmTileParams
    {
        uint32_t    m, n, k;
        const char* a;
        const char* b;
        const char* c;
        char*       d;
        uint32_t    lda, ldb, ldc, ldd; // elements
        double      alpha, beta; // narrowed to the accumulator type in the epilogue
        uint32_t    tilesM, tilesN;
        // the launch covers tile indices [tileFirst, tileFirst + tileCount) of the tilesM x tilesN walk; with
        // tileQuad the walk is over tiles of twice the kernel's edge, four workgroups each (tile_map.hpp)
        uint32_t tileFirst, tileCount, tileQuad;
        // split-K (128 x 128 tile kernels): workgroup row blockIdx.y multiplies K stages [y * splitStages, (y + 1) * splitStages)
        // and writes its partial D (in the accumulator type) at d + y * splitStrideD bytes; 0 = the whole K in one workgroup
        uint32_t splitStages;
        uint64_t splitStrideD;
        // host side only: 16-bit operands on the 256 x 256 tile take the five-buffer K loop instead of the two-buffer one
        uint32_t deepPipeline;
        // experiment (R355_STAGGER_TICKS in the environment, 10 ns units; 0 = off): the first staggerBlocks workgroups - the
        // first round over the CUs - start 0, 1, 2 or 3 x stagger ticks late, by groups of CUs within each XCD, so that
        // the rounds' epilogues do not all store at once
        uint32_t stagger, staggerBlocks;
    };
    // sum of `splits` partial results (accumulator type: f32, i32 or f64) + the alpha / beta epilogue into the output type
    int splitKReduce(const r355_gemm_args& g, const GemmTileParams& p, uint32_t splits, hipStream_t stream);
    // launch of one kernel family; aK / bK: operand is K-contiguous; tile: 256 or 128
    int gemmTiledPart0(const r355_gemm_args& g, bool aK, bool bK, uint32_t tile, const GemmTileParams& p, hipStream_t s);
    int gemmTiledPart1(const r355_gemm_args& g, bool aK, bool bK, uint32_t tile, const GemmTileParams& p, hipStream_t s);
    int gemmTiledPart2(const r355_gemm_args& g, bool aK, bool bK, uint32_t tile, const GemmTileParams& p, hipStream_t s);
    int gemmTiledPart3(const r355_gemm_args& g, bool aK, bool bK, uint32_t tile, const GemmTileParams& p, hipStream_t s);
} // namespace r355

namespace
{
    using i32x4  = int __attribute__((ext_vector_type(4)));
    using i32x2  = int __attribute__((ext_vector_type(2)));
    using f16x8  = _Float16 __attribute__((ext_vector_type(8)));
    using bf16x8 = __bf16 __attribute__((ext_vector_type(8)));
    typedef __fp16 trv4 __attribute__((__vector_size__(4 * sizeof(__fp16)))); // operand type of the transposing LDS read

    enum class Elem
    {
        F16,
        BF16,
        E4M3,
        I8,
        F32,
        F64,
        E5M2
    };

    constexpr uint32_t TILE_M      = 256;
    constexpr uint32_t TILE_N      = 256;
    constexpr uint32_t STAGE_KB    = 128; // bytes of K per stage per row
    constexpr uint32_t OPER_BYTES  = TILE_M * STAGE_KB; // 32 KiB per operand per stage
    constexpr uint32_t STAGE_BYTES = 2 * OPER_BYTES;
    constexpr uint32_t NUM_STAGES  = 2; // 16-bit kernel
    constexpr uint32_t THREADS     = 256;
    constexpr uint32_t CHUNK       = 16; // bytes moved per lane per access
    constexpr uint32_t LOADS_PER_OPER = OPER_BYTES / CHUNK / THREADS; // 8

    template <Elem E>
    struct ElemTraits;
    template <>
    struct ElemTraits<Elem::F16>
    {
        static constexpr uint32_t Bytes = 2;
    };
    template <>
    struct ElemTraits<Elem::BF16>
    {
        static constexpr uint32_t Bytes = 2;
    };
    template <>
    struct ElemTraits<Elem::E4M3>
    {
        static constexpr uint32_t Bytes = 1;
    };
    template <>
    struct ElemTraits<Elem::I8>
    {
        static constexpr uint32_t Bytes = 1;
    };
    template <>
    struct ElemTraits<Elem::F32>
    {
        static constexpr uint32_t Bytes = 4;
    };
    template <>
    struct ElemTraits<Elem::F64>
    {
        static constexpr uint32_t Bytes = 8;
    };
    template <>
    struct ElemTraits<Elem::E5M2>
    {
        static constexpr uint32_t Bytes = 1;
    };

    using Params = r355::GemmTileParams;

    __device__ __forceinline__ void staggeredStart(const Params& p)
    {
        if(p.stagger != 0u && blockIdx.x < p.staggerBlocks)
        {
            const uint32_t group = (blockIdx.x >> 3) & 3u; // workgroup ids go round the 8 XCDs: four groups of CUs in each
            const uint64_t until = __builtin_amdgcn_s_memrealtime() + (uint64_t)group * p.stagger; // 100 MHz counter
            while(__builtin_amdgcn_s_memrealtime() < until)
                __builtin_amdgcn_s_sleep(8);
        }
    }

    // The share of a split-K workgroup row: operands advanced to its first K stage, k cut to its stages, D pointed at its
    // partial result.  kStage: bytes between K stages of A / B (128 for a K-contiguous operand, 128 rows of ld otherwise).
    template <uint32_t ES>
    __device__ __forceinline__ Params splitShare(const Params& in, uint64_t kStageA, uint64_t kStageB)
    {
        Params p = in;
        if(in.splitStages != 0u)
        {
            const uint32_t y = blockIdx.y, first = y * in.splitStages; // first K stage of this share
            p.a += first * kStageA;
            p.b += first * kStageB;
            const uint32_t kFirst = first * (STAGE_KB / ES); // elements
            const uint32_t kShare = in.splitStages * (STAGE_KB / ES);
            p.k = in.k - kFirst < kShare ? in.k - kFirst : kShare;
            p.d += y * in.splitStrideD;
        }
        return p;
    }

    // ------------------------------------------------------------------------------------------
    // f16 / bf16 on v_mfma_f32_16x16x32_{f16,bf16}.
    //   * wave tile 128 x 128 = 8 x 8 accumulators of 4 registers; a stage is two K steps of 32;
    //     the operands of one K step (8 + 8 blocks, 128 registers for both steps) are fetched one step
    //     ahead of their use;
    //   * lane -> operand mapping: row lane % 16, 16-byte chunk lane / 16 of the 64-byte K step;
    //   * K-contiguous tile in LDS: 256 rows x 128 B, chunk c of row r in slot c ^ ((r >> 1) & 7): 16
    //     consecutive rows of one chunk index cover all 64 banks once;
    //   * M/N-contiguous tile in LDS: 64 k-rows x 512 B; a 32-lane transposing read covers k-rows 0..3
    //     and 8..11 times 32 bytes, so the swizzle depends on bits 0, 1 and 3 of the k-row, which makes
    //     the global -> LDS lane offset alternate between two values from one load to the next;
    //   * accumulator block (i, j): lane holds D(16 i + lane % 16, 16 j + 4 (lane / 16) + 0..3).
    using f32x4 = float __attribute__((ext_vector_type(4)));

    // The compiler selects these 4-register-result instructions with a destination that is not tied
    // to the C operand, and its register allocator then moves the 64 accumulators around inside the K
    // loop (thousands of copies).  Written as inline assembly the accumulator is updated in place, in an
    // AGPR.  The price: the compiler no longer knows these are matrix instructions, so the K loop below
    // fixes the instruction order itself, and the epilogue waits out the result latency by hand.
    template <Elem E>
    __device__ __forceinline__ void mfma16(f32x4& acc, i32x4 x, i32x4 y)
    {
        if constexpr(E == Elem::F16)
            asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(x), "v"(y));
        else
            asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(x), "v"(y));
    }

    // K tails.  A K stage with only `valid` (< 128) bytes of K left per row is completed with zeros by the
    // loads themselves: a buffer load whose offset lies outside its buffer writes zeros to LDS.  For an
    // M/N-contiguous operand the buffer of a stage ends after its last valid k-row (`valid` bytes of K are
    // valid / element size rows of ld elements: valid * ld bytes; the range check of a raw buffer on this
    // hardware covers lane offset + scalar offset); a K-contiguous lane whose chunk lies beyond K uses an
    // offset no buffer contains.
    __device__ __forceinline__ uint32_t stageRecords(bool kContig, uint32_t valid, uint32_t ld)
    {
        return kContig ? 0x7FFFFFFFu : valid * ld;
    }
    __device__ __forceinline__ i32x4 stageRsrc8(bool kContig, uint64_t addr, uint32_t valid, uint32_t ld)
    {
        return i32x4{static_cast<int>(static_cast<uint32_t>(addr)), static_cast<int>(static_cast<uint32_t>(addr >> 32) & 0xFFFFu),
                     static_cast<int>(stageRecords(kContig, valid, ld)), 0x00020000};
    }
    __device__ __forceinline__ uint32_t tailOffset(bool kContig, uint32_t laneOffset, uint32_t kByte, uint32_t valid)
    {
        return kContig && kByte >= valid ? 0x80000000u : laneOffset;
    }

    // D = alpha * acc + beta * C for one wave's tile of WB x WB accumulator blocks (16 x 16 each), row-major;
    // the wave tile starts at (m0, n0).  `scratch` is WB * 4 KiB of LDS owned by this wave.
    //
    // A lane holds four consecutive columns of one row of every block.  The tile is transposed through the wave's own LDS,
    // 128 to 16 rows at a time, so that an access to C or D covers whole rows of the wave tile (128 to 512 bytes) with up
    // to 128 bits per lane.  What is staged: alpha * acc in the output type when beta is zero; in the compute type
    // otherwise, so that alpha * acc + beta * C is rounded once, as the reference's epilogue rounds it
    // (test/reference_impl.hpp:71-77).  C and D are reached through raw buffers that end with the tile's last valid row,
    // and a lane whose columns lie beyond n uses an offset no buffer contains: no branch around any access, so a pass's
    // reads of C are all requested before its part of the tile goes through LDS, its stores all follow their LDS reads in
    // batches, and no wait is for more than it needs.  (With a branch around every guarded access each store waited for
    // everything before it: beta != 0 cost 12 % (f16) to 25 % (e4m3) of an 8192^3 launch instead of the 4 - 13 % that
    // reading C takes.)  C may alias D: every element's C is read before its D is written, and passes, waves and
    // workgroups own disjoint rows and columns.
    // The wave tile is WBM x WBN blocks (rows x columns of 16 x 16) and `scratch` SCRATCH bytes of LDS owned by this wave.
    template <typename StageT, bool WITH_C, typename AccV, typename OutT, uint32_t WBM, uint32_t WBN, uint32_t SCRATCH>
    __device__ __forceinline__ void storeTileStaged(AccV (&acc)[WBM][WBN], const Params& p, uint32_t m0, uint32_t n0, uint32_t lane,
                                                    char* scratch)
    {
        using AccE = std::remove_reference_t<decltype(acc[0][0][0])>;
        const AccE     alpha = static_cast<AccE>(p.alpha), beta = static_cast<AccE>(p.beta);
        const uint32_t r16 = lane & 15u, g = lane >> 4;
        constexpr uint32_t SS = sizeof(StageT), OS = sizeof(OutT);
        constexpr uint32_t ROW_BYTES  = 16u * WBN * SS;
        constexpr uint32_t ROW_CHUNKS = ROW_BYTES / CHUNK; // 8, 16 or 32
        constexpr uint32_t SWZ        = ROW_CHUNKS < 16u ? ROW_CHUNKS - 1u : 15u;
        constexpr uint32_t EPC        = CHUNK / SS; // elements of a staged 16-byte chunk
        constexpr uint32_t OUT_WORDS  = EPC * OS / 4u; // 32-bit words of C and of D per lane and chunk: 4, 2 or 1
        // rows per pass: what the scratch holds, halved where a pass's part of C would take 128 registers
        constexpr uint32_t FIT_ALL    = SCRATCH / ROW_BYTES;
        constexpr uint32_t FIT        = FIT_ALL / ((WITH_C && FIT_ALL * ROW_CHUNKS / 64u * OUT_WORDS >= 128u) ? 2u : 1u);
        constexpr uint32_t ROWS_PASS  = FIT < 16u * WBM ? FIT : 16u * WBM;
        constexpr uint32_t BLOCKS_I   = ROWS_PASS / 16u; // row blocks per pass
        constexpr uint32_t ITERS      = ROWS_PASS * ROW_CHUNKS / 64u; // chunks per lane and pass
        constexpr uint32_t BATCH      = ITERS < 8u ? ITERS : 8u;
        constexpr int      NT         = 2; // cache policy of the raw buffer accesses: nontemporal (C is read, D written, once)
        static_assert(EPC * OS % 4u == 0u && ITERS % BATCH == 0u, "whole words per lane, whole batches per pass");

        const uint32_t lddB = p.ldd * OS, ldcB = p.ldc * OS;
        const uint32_t um0 = __builtin_amdgcn_readfirstlane(m0), un0 = __builtin_amdgcn_readfirstlane(n0); // (wave-uniform)
        const uint32_t colsValid = un0 < p.n ? (p.n - un0 < 16u * WBN ? p.n - un0 : 16u * WBN) : 0u;
        auto tileBuffer = [&](const char* base, uint32_t ldB, uint32_t rowFirst) {
            // from the wave tile's first column in row rowFirst to the end of the tile's last valid row (nothing if there is none)
            const uint32_t rowsLeft  = rowFirst < p.m ? p.m - rowFirst : 0u;
            const uint32_t rowsValid = rowsLeft < ROWS_PASS ? rowsLeft : ROWS_PASS;
            const uint32_t records   = (rowsValid && colsValid) ? (rowsValid - 1u) * ldB + colsValid * OS : 0u;
            const uint64_t addr      = reinterpret_cast<uint64_t>(base) + ((uint64_t)rowFirst * ldB + (uint64_t)un0 * OS);
            const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(addr));
            const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(addr >> 32));
            return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<char*>((static_cast<uint64_t>(hi) << 32) | lo), 0,
                                                     static_cast<int>(__builtin_amdgcn_readfirstlane(records)), 0x00020000);
        };
        // (lane offset + wave-uniform offset: the range check covers their sum)
        auto loadWords = [](__amdgpu_buffer_rsrc_t rsrc, uint32_t off, uint32_t uni, uint32_t (&w)[OUT_WORDS]) {
            if constexpr(OUT_WORDS == 4u)
            {
                const auto v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, uni, NT);
                w[0] = v[0], w[1] = v[1], w[2] = v[2], w[3] = v[3];
            }
            else if constexpr(OUT_WORDS == 2u)
            {
                const auto v = __builtin_amdgcn_raw_buffer_load_b64(rsrc, off, uni, NT);
                w[0] = v[0], w[1] = v[1];
            }
            else
                w[0] = __builtin_amdgcn_raw_buffer_load_b32(rsrc, off, uni, NT);
        };
        // A store's wave-uniform offset is added to the lane offset, not handed over as a scalar offset: after a store of
        // more than 64 bits whose offset field names a scalar register the compiler leaves no wait state before the next
        // write of the data registers (the hazard is documented for the other offset forms only), and this hardware then
        // stored the new value of the second data register now and then -- seen as an address word in D, a few times per
        // thousand wave tiles, when the instruction after the store recomputed that register.
        auto storeWords = [](__amdgpu_buffer_rsrc_t rsrc, uint32_t off, uint32_t uni, const uint32_t (&w)[OUT_WORDS]) {
            using u32x4 = uint32_t __attribute__((ext_vector_type(4)));
            using u32x2 = uint32_t __attribute__((ext_vector_type(2)));
            if constexpr(OUT_WORDS == 4u)
                __builtin_amdgcn_raw_buffer_store_b128(u32x4{w[0], w[1], w[2], w[3]}, rsrc, off + uni, 0, NT);
            else if constexpr(OUT_WORDS == 2u)
                __builtin_amdgcn_raw_buffer_store_b64(u32x2{w[0], w[1]}, rsrc, off + uni, 0, NT);
            else
                __builtin_amdgcn_raw_buffer_store_b32(w[0], rsrc, off + uni, 0, NT);
        };
        // chunk `it` of a lane: row it * RPI + lane / ROW_CHUNKS of the pass, 16-byte chunk lane % ROW_CHUNKS of the staged row
        constexpr uint32_t RPI = 64u / ROW_CHUNKS;
        const uint32_t rowLane = lane / ROW_CHUNKS, cLane = lane % ROW_CHUNKS;
        const bool     colOk   = cLane * EPC < colsValid;
        const uint32_t dLane = colOk ? rowLane * lddB + cLane * (EPC * OS) : 0x80000000u;

#pragma unroll
        for(uint32_t pass = 0; pass < WBM / BLOCKS_I; ++pass)
        {
            const auto dBuf = tileBuffer(p.d, lddB, um0 + pass * ROWS_PASS);
            // C of this pass, requested before anything else (m and n are multiples of 16, so a chunk of up to 16 elements
            // is inside the matrix or outside as a whole)
            uint32_t cWords[WITH_C ? ITERS : 1u][OUT_WORDS];
            if constexpr(WITH_C)
            {
                const auto     cBuf  = tileBuffer(p.c, ldcB, um0 + pass * ROWS_PASS);
                const uint32_t cLaneOff = colOk ? rowLane * ldcB + cLane * (EPC * OS) : 0x80000000u;
#pragma unroll
                for(uint32_t it = 0; it < ITERS; ++it)
                    loadWords(cBuf, cLaneOff, it * RPI * ldcB, cWords[it]);
            }
#pragma unroll
            for(uint32_t ii = 0; ii < BLOCKS_I; ++ii)
            {
                const uint32_t i = pass * BLOCKS_I + ii, row = 16u * ii + r16;
#pragma unroll
                for(uint32_t j = 0; j < WBN; ++j)
                {
                    if constexpr(sizeof(AccE) == 8)
                    {
                        // f64 accumulators: element e is column 4 e + lane / 16 of the block
#pragma unroll
                        for(uint32_t e = 0; e < 4; ++e)
                        {
                            const uint32_t byteInRow = (16u * j + 4u * e + g) * SS;
                            const uint32_t c = byteInRow / CHUNK, within = byteInRow % CHUNK;
                            *reinterpret_cast<StageT*>(scratch + row * ROW_BYTES + ((c ^ (row & SWZ)) * CHUNK) + within)
                                = static_cast<StageT>(alpha * acc[i][j][e]);
                        }
                    }
                    else
                    {
                        using StageV = StageT __attribute__((ext_vector_type(4)));
                        StageV out;
#pragma unroll
                        for(uint32_t e = 0; e < 4; ++e)
                            out[e] = static_cast<StageT>(alpha * acc[i][j][e]);
                        // 16 consecutive rows take 16 (8) different chunk slots
                        const uint32_t byteInRow = (16u * j + 4u * g) * SS;
                        const uint32_t c = byteInRow / CHUNK, within = byteInRow % CHUNK;
                        *reinterpret_cast<StageV*>(scratch + row * ROW_BYTES + ((c ^ (row & SWZ)) * CHUNK) + within) = out;
                    }
                }
            }
            __builtin_amdgcn_wave_barrier(); // the same wave reads back what it wrote (LDS is in order per wave)
#pragma unroll
            for(uint32_t b0 = 0; b0 < ITERS; b0 += BATCH)
            {
                union
                {
                    i32x4  v;
                    StageT s[EPC];
                } staged[BATCH];
#pragma unroll
                for(uint32_t u = 0; u < BATCH; ++u)
                {
                    const uint32_t row = (b0 + u) * RPI + rowLane;
                    staged[u].v = *reinterpret_cast<const i32x4*>(scratch + row * ROW_BYTES + ((cLane ^ (row & SWZ)) * CHUNK));
                }
#pragma unroll
                for(uint32_t u = 0; u < BATCH; ++u)
                {
                    union
                    {
                        uint32_t w[OUT_WORDS];
                        OutT     o[EPC];
                    } res;
                    if constexpr(WITH_C)
                    {
                        union
                        {
                            uint32_t w[OUT_WORDS];
                            OutT     o[EPC];
                        } cin;
#pragma unroll
                        for(uint32_t w = 0; w < OUT_WORDS; ++w)
                            cin.w[w] = cWords[b0 + u][w];
#pragma unroll
                        for(uint32_t e = 0; e < EPC; ++e)
                            res.o[e] = static_cast<OutT>(static_cast<AccE>(staged[u].s[e]) + beta * static_cast<AccE>(cin.o[e]));
                    }
                    else
                    {
                        static_assert(WITH_C || sizeof(StageT) == sizeof(OutT), "staged in the output type when beta is zero");
#pragma unroll
                        for(uint32_t w = 0; w < OUT_WORDS; ++w)
                            res.w[w] = static_cast<uint32_t>(staged[u].v[w]);
                    }
                    storeWords(dBuf, dLane, (b0 + u) * RPI * lddB, res.w);
                }
            }
            __builtin_amdgcn_wave_barrier();
        }
    }

    // (`scratch`: WB x 4 KiB of the wave's own; the eight-wave kernel has 16 KiB for its 8 x 4 blocks)
    template <typename AccV, typename OutT, uint32_t WBM, uint32_t WBN, uint32_t SCRATCH = WBM * 4096u>
    __device__ __forceinline__ void storeTile16(AccV (&acc)[WBM][WBN], const Params& p, uint32_t m0, uint32_t n0, uint32_t lane,
                                                char* scratch)
    {
        using AccE = std::remove_reference_t<decltype(acc[0][0][0])>;
        if(static_cast<AccE>(p.beta) == static_cast<AccE>(0)) // (as the accumulator type sees it: an int8 problem's beta = 0.5 is 0)
            storeTileStaged<OutT, false, AccV, OutT, WBM, WBN, SCRATCH>(acc, p, m0, n0, lane, scratch);
        else
            storeTileStaged<AccE, true, AccV, OutT, WBM, WBN, SCRATCH>(acc, p, m0, n0, lane, scratch);
    }

    //
    // WB is the number of accumulator blocks per wave tile edge: 8 (wave tile 128 x 128, macro tile
    // 256 x 256, one workgroup per CU).  The body also works with 4 (wave tile 64 x 64, macro tile
    // 128 x 128, 64 KiB of LDS), but the small tile is served by the five-buffer body further down, which
    // keeps more loads in flight.
    template <Elem E, typename OutT, bool A_KCONTIG, bool B_KCONTIG, uint32_t WB>
    __device__ __forceinline__ void gemmTiled16(const Params& p)
    {
        constexpr uint32_t ES = ElemTraits<E>::Bytes;
        constexpr uint32_t TK = STAGE_KB / ES; // 64 K elements per stage = two K steps of 32
        static_assert(ES == 2, "16-bit element types only");
        static_assert(WB == 8 || WB == 4, "wave tile of 8 x 8 or 4 x 4 blocks");
        R355_STAMP(0);
        R355_STAMP_ID();
        constexpr uint32_t TILE  = 32u * WB; // macro tile edge
        constexpr uint32_t WT    = 16u * WB; // wave tile edge
        constexpr uint32_t OPER  = TILE * STAGE_KB; // bytes of one operand per stage
        constexpr uint32_t LOADS = OPER / CHUNK / THREADS; // direct loads per operand per stage = WB
        constexpr uint32_t ROWB  = TILE * ES; // bytes of a k-row of an M/N-contiguous operand tile
        constexpr uint32_t KROWS = THREADS * CHUNK / ROWB; // k-rows of such a tile one load covers: 8 or 16
        constexpr uint32_t XS    = 2u * WB; // operand blocks per K step
        constexpr uint32_t QS    = WB / 2u; // matrix instructions per operand block

        // One variable per stage: the compiler tracks outstanding direct-to-LDS loads per LDS variable.
        __shared__ __attribute__((aligned(1024))) char stage0[2u * OPER];
        __shared__ __attribute__((aligned(1024))) char stage1[2u * OPER];

        uint32_t tm, tn;
        if(!r355::tileCoordRange(blockIdx.x, p.tilesM, p.tilesN, p.tileFirst, p.tileCount, p.tileQuad != 0u, tm, tn))
            return;
        if(p.tileQuad && (tm * TILE >= p.m || tn * TILE >= p.n))
            return; // a quarter of a partial edge tile that lies outside the matrix
        staggeredStart(p);

        const uint32_t tid  = threadIdx.x;
        const uint32_t lane = tid & 63u;
        const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const uint32_t wm = wave >> 1, wn = wave & 1u;
        auto           swzK  = [](uint32_t row) { return (row >> 1) & 7u; };
        auto           swzMN = [](uint32_t krow) { return ((krow & 3u) << 2) | (((krow >> 3) & 1u) << 1); };

        // ---------------- global -> LDS: chunk L = j * 256 + tid of an operand tile sits at LDS byte 16 L.
        // K-contiguous: row L / 8, and the swizzle does not change with j (32 rows per load).
        // M/N-contiguous: k-row L / (ROWB / 16) = KROWS j + tid / (ROWB / 16); with 8 k-rows per load the
        // swizzle alternates with bit 3 of the k-row.
        // Edge tiles (m or n not a multiple of 256) must not read outside the operands: a lane whose
        // row (K-contiguous) or 16-byte chunk (M/N-contiguous) lies beyond the matrix reads the last valid
        // row / the first chunk instead -- what lands in LDS for it only feeds elements of D that are
        // never stored.  Hence one lane offset per load (the compiler merges equal ones).
        uint32_t       gOffA[LOADS], gOffB[LOADS], gStepA, gStepB; // gStep: uniform offset per load
        uint32_t       kByteA = 0u, kByteB = 0u; // K-contiguous: K offset inside a stage of this lane's chunks
        uint64_t       gStageA, gStageB; // bytes between consecutive K stages
        const uint32_t validM = p.m - tm * TILE < TILE ? p.m - tm * TILE : TILE;
        const uint32_t validN = p.n - tn * TILE < TILE ? p.n - tn * TILE : TILE;
        auto laneOffsets = [&](bool kContig, uint32_t ld, uint32_t valid, uint32_t (&off)[LOADS], uint32_t& step,
                               uint64_t& stage, uint32_t& kByte) {
            if(kContig)
            {
                const uint32_t r = tid >> 3, slot = tid & 7u;
                kByte = (slot ^ swzK(r)) * CHUNK;
#pragma unroll
                for(uint32_t j = 0; j < LOADS; ++j)
                {
                    const uint32_t row = r + 32u * j < valid ? r + 32u * j : valid - 1u;
                    off[j]             = row * ld * ES + ((slot ^ swzK(r)) * CHUNK);
                }
                step = 0u, stage = STAGE_KB;
            }
            else
            {
                constexpr uint32_t SLOTS = ROWB / CHUNK; // 32 or 16 chunks per k-row
                const uint32_t     r = tid / SLOTS, slot = tid % SLOTS;
#pragma unroll
                for(uint32_t j = 0; j < LOADS; ++j)
                {
                    const uint32_t c = slot ^ swzMN(r + KROWS * j);
                    off[j]           = r * ld * ES + (c * (CHUNK / ES) < valid ? c : 0u) * CHUNK;
                }
                step = KROWS * ld * ES, stage = (uint64_t)TK * ld * ES;
            }
        };
        laneOffsets(A_KCONTIG, p.lda, validM, gOffA, gStepA, gStageA, kByteA);
        laneOffsets(B_KCONTIG, p.ldb, validN, gOffB, gStepB, gStageB, kByteB);
        const char* gA = p.a + (A_KCONTIG ? (uint64_t)tm * TILE * p.lda * ES : (uint64_t)tm * TILE * ES);
        const char* gB = p.b + (B_KCONTIG ? (uint64_t)tn * TILE * p.ldb * ES : (uint64_t)tn * TILE * ES);

        // ---------------- LDS -> registers (per lane, fixed)
        // K-contiguous: block i rows are 16 i + lane % 16; K step s reads chunk 4 s + lane / 16.
        // M/N-contiguous: K step s, half h: k-row 32 s + 8 (lane / 16) + 4 h + (lane % 16) / 4,
        //                 8-byte piece m / 4 with m = 16 i + 4 (lane % 4).
        uint32_t rdA[WB], rdB[WB];
        const uint32_t t = lane & 15u, g = lane >> 4;
        if constexpr(A_KCONTIG)
        {
            const uint32_t r = wm * WT + t;
            rdA[0] = r * STAGE_KB + ((g ^ swzK(r)) * CHUNK);
            rdA[1] = r * STAGE_KB + (((4u + g) ^ swzK(r)) * CHUNK);
        }
        else
        {
            const uint32_t kr = 8u * g + (t >> 2);
#pragma unroll
            for(uint32_t i = 0; i < WB; ++i)
            {
                const uint32_t piece = wm * (WT / 4u) + 4u * i + (t & 3u);
                rdA[i] = kr * ROWB + (((piece >> 1) ^ swzMN(kr)) * CHUNK) + (piece & 1u) * 8u;
            }
        }
        if constexpr(B_KCONTIG)
        {
            const uint32_t r = wn * WT + t;
            rdB[0] = OPER + r * STAGE_KB + ((g ^ swzK(r)) * CHUNK);
            rdB[1] = OPER + r * STAGE_KB + (((4u + g) ^ swzK(r)) * CHUNK);
        }
        else
        {
            const uint32_t kr = 8u * g + (t >> 2);
#pragma unroll
            for(uint32_t i = 0; i < WB; ++i)
            {
                const uint32_t piece = wn * (WT / 4u) + 4u * i + (t & 3u);
                rdB[i] = OPER + kr * ROWB + (((piece >> 1) ^ swzMN(kr)) * CHUNK) + (piece & 1u) * 8u;
            }
        }
        // An operand block arrives in one 128-bit read (part 0) or in two transposing 64-bit reads
        // (parts 0 and 1, the low and high four K values of each lane).
        using lpt = __attribute__((address_space(3))) trv4*;
        auto readA = [&](const char* base, uint32_t i, uint32_t s, uint32_t part, i32x4& dst) {
            if constexpr(A_KCONTIG)
            {
                if(part == 0u)
                    dst = *reinterpret_cast<const i32x4*>(base + rdA[s] + i * 16u * STAGE_KB);
            }
            else
            {
                const char* q = base + rdA[i] + s * 32u * ROWB + part * 4u * ROWB;
                const i32x2 v = __builtin_bit_cast(i32x2, __builtin_amdgcn_ds_read_tr16_b64_v4f16((lpt)q));
                dst[2u * part] = v[0], dst[2u * part + 1u] = v[1];
            }
        };
        auto readB = [&](const char* base, uint32_t i, uint32_t s, uint32_t part, i32x4& dst) {
            if constexpr(B_KCONTIG)
            {
                if(part == 0u)
                    dst = *reinterpret_cast<const i32x4*>(base + rdB[s] + i * 16u * STAGE_KB);
            }
            else
            {
                const char* q = base + rdB[i] + s * 32u * ROWB + part * 4u * ROWB;
                const i32x2 v = __builtin_bit_cast(i32x2, __builtin_amdgcn_ds_read_tr16_b64_v4f16((lpt)q));
                dst[2u * part] = v[0], dst[2u * part + 1u] = v[1];
            }
        };

        // ---------------- global -> LDS, written by the memory pipeline: 16 loads per stage
        // wave-uniform addresses are kept as integers the compiler can see are uniform
        auto uniform64 = [](const char* ptr) {
            const uint64_t v  = reinterpret_cast<uint64_t>(ptr);
            const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
            const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
            return (static_cast<uint64_t>(hi) << 32) | lo;
        };
        // K stages come in pairs; K need not fill the last pair: stage st holds validOf(st) = 0 .. 128 valid
        // bytes per row and the loads fill the rest with zeros
        const uint32_t kBytes    = p.k * ES;
        const uint32_t numStages = (kBytes + 2u * STAGE_KB - 1u) / (2u * STAGE_KB) * 2u;
        auto           validOf   = [&](uint32_t st) { // 0 for the padding stage and for refills past the end: no traffic
            return st * STAGE_KB >= kBytes ? 0u : (kBytes - st * STAGE_KB < STAGE_KB ? kBytes - st * STAGE_KB : STAGE_KB);
        };
        auto rsrcAt = [](uint64_t addr, uint32_t records) { // raw buffer, 32-bit data format, no swizzle
            return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<char*>(addr), 0, static_cast<int>(records), 0x00020000);
        };
        // load x of a stage with vA / vB valid bytes of K: x = 2 j loads piece j of A, x = 2 j + 1 piece j of B.  `full`
        // (a compile-time tag): the stage is known to be a whole one, so no lane has a chunk beyond K and the lane offsets
        // are used as they are - the K loop's main part carries no select per load.
        auto issueLoad = [&](auto full, __amdgpu_buffer_rsrc_t srcA, __amdgpu_buffer_rsrc_t srcB, uint32_t vA, uint32_t vB,
                             char* stage, uint32_t x) {
            using lp         = __attribute__((address_space(3))) void*;
            constexpr bool FULL = decltype(full)::value;
            const uint32_t j = x >> 1;
            char*          dst = stage + (j * THREADS + wave * 64u) * CHUNK;
            if(x & 1u)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(srcB, (lp)(dst + OPER), 16,
                                                         FULL ? gOffB[j] : tailOffset(B_KCONTIG, gOffB[j], kByteB, vB), j * gStepB, 0, 0);
            else
                __builtin_amdgcn_raw_ptr_buffer_load_lds(srcA, (lp)dst, 16,
                                                         FULL ? gOffA[j] : tailOffset(A_KCONTIG, gOffA[j], kByteA, vA), j * gStepA, 0, 0);
        };
        auto issueGlobal = [&](uint32_t kt, char* stage) {
            const uint32_t               v    = validOf(kt);
            const __amdgpu_buffer_rsrc_t srcA = rsrcAt(uniform64(gA + kt * gStageA), stageRecords(A_KCONTIG, v, p.lda)),
                                         srcB = rsrcAt(uniform64(gB + kt * gStageB), stageRecords(B_KCONTIG, v, p.ldb));
#pragma unroll
            for(uint32_t x = 0; x < 2u * LOADS; ++x)
                issueLoad(std::false_type{}, srcA, srcB, v, v, stage, x);
        };

        f32x4          acc[WB][WB];
#pragma unroll
        for(uint32_t i = 0; i < WB; ++i)
#pragma unroll
            for(uint32_t j = 0; j < WB; ++j)
                acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

        i32x4    fa[2][WB], fb[2][WB];
        uint64_t refillA, refillB; // where the next refill reads from (stage kt + 2, clamped to the last stage)
        // Matrix instruction n (0 .. WB * WB - 1) of a K step works on accumulator block (i, j) = blockOf(n): block
        // row / column d is first needed after d * d instructions, and the operands arrive in the
        // order A0 B0 A1 B1 ...  Operands swapped: each lane then holds 4 consecutive columns of a row of D.
        auto mfmaAt = [&](uint32_t s, uint32_t n) {
            uint32_t d = 0;
            while((d + 1u) * (d + 1u) <= n)
                ++d;
            const uint32_t r = n - d * d; // 0..2d within the L-shaped shell d
            const uint32_t i = r <= d ? d : r - d - 1u, j = r <= d ? r : d;
            mfma16<E>(acc[i][j], fb[s][j], fa[s][i]);
        };
        // operand block x of K step s: x = 2 i is A block i, x = 2 i + 1 is B block i
        auto readAt = [&](const char* base, uint32_t s, uint32_t x, uint32_t part) {
            if(x & 1u)
                readB(base, x >> 1, s, part, fb[s][x >> 1]);
            else
                readA(base, x >> 1, s, part, fa[s][x >> 1]);
        };
        auto readStep = [&](const char* base, uint32_t s) {
#pragma unroll
            for(uint32_t x = 0; x < XS; ++x)
            {
                readAt(base, s, x, 0);
                readAt(base, s, x, 1);
            }
        };

        // One K stage; `cur` / `nxt` are the LDS buffers of stage kt / kt + 1.  K step 0 is in registers:
        // step 1 arrives under its matrix instructions; then every wave holds the rest of `cur` in
        // registers, so after the barrier `cur` is refilled with stage kt + 2 while step 0 of stage
        // kt + 1 arrives from `nxt` under the matrix instructions of step 1.  A matrix instruction
        // occupies its pipeline for 16 cycles and the wave can issue about three other instructions
        // in that time, so the other work is dealt out one piece per matrix instruction, in groups of
        // four: read (part 0), read (part 1), direct load (second step), nothing -- and nothing moves
        // between pieces (groups of two with the small wave tile: read, read + direct load).  Every stage
        // runs the same code: past the end the refill has nothing in range (it writes zeros) and the operands read
        // ahead are never used.
        // `full` (compile-time tag): the stage this one refills (kt + 2) and the one after it are whole stages inside K - the
        // main part of the K loop, whose loads then carry no tail select and whose refill pointers always advance.
        constexpr uint32_t LOAD_Q = QS > 2u ? 2u : QS - 1u;
        auto stageBody = [&](auto full, uint32_t kt, char* cur, char* nxt) {
            constexpr bool FULL = decltype(full)::value;
#pragma unroll
            for(uint32_t x = 0; x < XS; ++x)
            {
#pragma unroll
                for(uint32_t q = 0; q < QS; ++q)
                {
                    mfmaAt(0, QS * x + q);
                    if(q < 2u)
                        readAt(cur, 1, x, q);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): stage kt + 1 has landed
            __syncthreads();
            const uint32_t               v    = FULL ? STAGE_KB : validOf(kt + 2u);
            const __amdgpu_buffer_rsrc_t srcA = rsrcAt(refillA, stageRecords(A_KCONTIG, v, p.lda)),
                                         srcB = rsrcAt(refillB, stageRecords(B_KCONTIG, v, p.ldb));
            if(FULL || kt + 3u < numStages) // the refill of the next stage is one stage further, or the last again
                refillA += gStageA, refillB += gStageB;
#pragma unroll
            for(uint32_t x = 0; x < XS; ++x)
            {
#pragma unroll
                for(uint32_t q = 0; q < QS; ++q)
                {
                    mfmaAt(1, QS * x + q);
                    if(q < 2u)
                        readAt(nxt, 0, x, q);
                    if(q == LOAD_Q)
                        issueLoad(full, srcA, srcB, v, v, cur, x);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        };

        // prologue: stage 0 resident, stage 1 in flight, first operands in registers
        issueGlobal(0, stage0);
        issueGlobal(1, stage1);
        __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0)
        __syncthreads();
        R355_STAMP(1);
        readStep(stage0, 0);
        refillA = uniform64(gA + (numStages > 2u ? 2u : numStages - 1u) * gStageA);
        refillB = uniform64(gB + (numStages > 2u ? 2u : numStages - 1u) * gStageB);

        // main part: every stage a pair refills (up to kt + 3) is a whole stage of K; then the pairs around the end of K
        // (only a K-contiguous operand has a select to lose: with none, the main part is empty and compiles away)
        const uint32_t wholeStages = (A_KCONTIG || B_KCONTIG) ? kBytes / STAGE_KB : 0u;
        uint32_t       kt          = 0;
        for(; kt + 3u < wholeStages; kt += 2)
        {
            stageBody(std::true_type{}, kt, stage0, stage1);
            stageBody(std::true_type{}, kt + 1, stage1, stage0);
        }
        for(; kt < numStages; kt += 2)
        {
            stageBody(std::false_type{}, kt, stage0, stage1);
            stageBody(std::false_type{}, kt + 1, stage1, stage0);
        }

        R355_STAMP(2);
        // the refills past the end (zeros) are still landing in the buffers the epilogue reuses
        __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0)
        __syncthreads();
        // the last matrix instructions are still in the pipeline and the compiler does not know it
        asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
        storeTile16<f32x4, OutT, WB, WB>(acc, p, tm * TILE + wm * WT, tn * TILE + wn * WT, lane,
                                     ((wave < 2u) ? stage0 : stage1) + (wave & 1u) * (WB * 4096u));
        R355_STAMP_END();
    }

    // (a waves-per-EU attribute that depends on a template parameter makes the compiler drop the host-side
    // launch stub without a diagnostic, hence separate kernels per tile size around common bodies)
    template <Elem E, typename OutT, bool A_KCONTIG, bool B_KCONTIG>
    __global__ void __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(1, 1))) gemmTiledKernel16(Params p)
    {
        gemmTiled16<E, OutT, A_KCONTIG, B_KCONTIG, 8>(p);
    }

    // ------------------------------------------------------------------------------------------
    // 8-bit operands (int8, e4m3), either orientation, and the small macro tile of every type: five LDS
    // buffers.  At twice the matrix-instruction rate (or a quarter of the tile) a K stage lasts about as
    // long as a direct load takes to arrive, so a two-buffer scheme leaves the memory pipe idle while a
    // refill waits for its consumer.  Here LDS
    // holds two buffers for A and three for B (5 x 32 KiB = all 160 KiB): the B half of a stage is
    // requested three stages ahead and the A half two, which keeps 96 KiB per CU in flight instead
    // of 64.  Stage kt lives in A buffer kt % 2 and B buffer kt % 3, so six stages bring every buffer
    // back to its starting role; the K loop is unrolled six times with a single exit (an exit after
    // every stage makes the register allocator spill hundreds of registers) and the up to five
    // remaining stages follow as straight-line code, so any number of stages runs.  Loads past the
    // last stage have nothing in range -- they write zeros into buffers nobody reads any more -- so every stage
    // issues the same 16 loads and the wait before its barrier is always "all but the youngest 8".
    //
    // The direct loads are inline assembly: for the builtin the compiler cannot tell which buffer a
    // later ds_read depends on and waits for vmcnt(0) every time, which would serialise exactly the
    // loads that are meant to stay in flight.  Issued this way the only vmcnt waits are the ones
    // written here.
    //
    // Operand tiles in LDS (32 KiB each), chunk L = j * 256 + tid of a tile at byte 16 L:
    //   * K-contiguous (A row-major / B col-major): 256 rows x 128 B, chunk c of row r in slot
    //     c ^ ((r >> 1) & 7); a lane reads 16 consecutive K bytes of its row with one ds_read_b128;
    //   * M/N-contiguous (A col-major / B row-major): 128 k-rows x 256 B, chunk c of k-row q in slot
    //     c ^ ((q & 7) | ((q >> 1) & 8)).  ds_read_b64_tr_b8 transposes inside each group of 16 lanes:
    //     lane t supplies the address of 8 bytes, k-row t / 2 and byte columns 8 (t % 2) .. + 7, and
    //     receives column t of the group's 8 k-rows -- 8 consecutive K values of one row of the operand,
    //     which is what the matrix instructions want.  Two such reads make the 16 K bytes a
    //     ds_read_b128 delivers for a K-contiguous operand.  The 32 lanes of one LDS pass touch 16
    //     k-rows (8 each from two lane groups, 16 k-rows apart), hence bit 4 in the swizzle.
    using r355::ldsBarrier;
    using r355::loadToLds;
    using r355::waitVmcnt;

    using r355::tile::laneOffsets8;
    using r355::tile::readBlock8;
    using r355::tile::readOffsets8;
    using r355::tile::swzK8;
    using r355::tile::swzMN8;

    // ------------------------------------------------------------------------------------------
    // int8 on v_mfma_i32_16x16x64_i8: the five-buffer scheme with the K-step structure and the
    // in-place inline-assembly accumulators of gemmTiledKernel16.  A stage is two
    // K steps of 64 bytes; lane -> operand mapping: row lane % 16, K bytes 16 (lane / 16) .. + 15 of the step.
    using i32x4v = int __attribute__((ext_vector_type(4)));
    __device__ __forceinline__ void mfma16i8(i32x4v& acc, i32x4 x, i32x4 y)
    {
        asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+a"(acc) : "v"(x), "v"(y));
    }

    // f32 on v_mfma_f32_16x16x4_f32: a lane's 16 bytes are four K values, consumed by four instructions
    // (instruction e multiplies element e of every lane: k = 4 (lane / 16) + e of each 16-wide K step)
    __device__ __forceinline__ void mfma16f32(f32x4& acc, i32x4 x, i32x4 y)
    {
#pragma unroll
        for(uint32_t e = 0; e < 4; ++e)
            asm volatile("v_mfma_f32_16x16x4_f32 %0, %1, %2, %0" : "+a"(acc) : "v"(x[e]), "v"(y[e]));
    }

    // f64 on v_mfma_f64_16x16x4_f64: a lane's 16 bytes are two K values (k = 2 (lane / 16) + e of each 8-wide K
    // step) for two instructions.  An accumulator block is 8 registers, so only the 4 x 4 wave tile fits; its
    // elements are rows lane / 16 + 4 e of column lane % 16 (with the operands swapped as everywhere here:
    // columns lane / 16 + 4 e of row lane % 16), unlike the four consecutive ones of the 32-bit accumulators.
    using f64x4 = double __attribute__((ext_vector_type(4)));
    __device__ __forceinline__ void mfma16f64(f64x4& acc, i32x4 x, i32x4 y)
    {
#pragma unroll
        for(uint32_t e = 0; e < 2; ++e)
        {
            const double xe = __builtin_bit_cast(double, i32x2{x[2u * e], x[2u * e + 1u]});
            const double ye = __builtin_bit_cast(double, i32x2{y[2u * e], y[2u * e + 1u]});
            asm volatile("v_mfma_f64_16x16x4_f64 %0, %1, %2, %0" : "+a"(acc) : "v"(xe), "v"(ye));
        }
    }

    template <Elem E, typename OutT, bool A_KCONTIG, bool B_KCONTIG, uint32_t WB>
    __device__ __forceinline__ void gemmTiled5(const Params& whole)
    {
        static_assert(WB == 8 || WB == 4, "wave tile of 8 x 8 or 4 x 4 blocks");
        static_assert(E != Elem::F64 || WB == 4, "f64 accumulators of an 8 x 8 wave tile would need 512 registers");
        static_assert(E != Elem::E4M3 && E != Elem::E5M2, "fp8 has its own stage structure");
        R355_STAMP(0);
        R355_STAMP_ID();
        constexpr uint32_t ES = ElemTraits<E>::Bytes;
        // split-K: this workgroup row's share of K (the whole problem when splitStages is 0)
        const Params p = splitShare<ES>(whole, A_KCONTIG ? (uint64_t)STAGE_KB : (uint64_t)STAGE_KB * whole.lda,
                                        B_KCONTIG ? (uint64_t)STAGE_KB : (uint64_t)STAGE_KB * whole.ldb);
        using AccV            = std::conditional_t<E == Elem::I8, i32x4v, std::conditional_t<E == Elem::F64, f64x4, f32x4>>;
        constexpr uint32_t TILE = 32u * WB, WT = 16u * WB; // macro tile and wave tile edge
        constexpr uint32_t OPER = TILE * STAGE_KB; // bytes of one operand per stage: 32 or 16 KiB
        constexpr uint32_t XS = 2u * WB, QS = WB / 2u; // operand blocks per K step, matrix instructions per block
        constexpr uint32_t LOAD_Q = QS > 2u ? 2u : QS - 1u;
        // LDS map: A buffers at 0 and OPER, B buffers at 2, 3 and 4 OPER
        constexpr uint32_t A_AT[2] = {0u, OPER};
        constexpr uint32_t B_AT[3] = {2u * OPER, 3u * OPER, 4u * OPER};
        __shared__ __attribute__((aligned(1024))) char lds[5u * OPER];

        uint32_t tm, tn;
        if(!r355::tileCoordRange(blockIdx.x, p.tilesM, p.tilesN, p.tileFirst, p.tileCount, p.tileQuad != 0u, tm, tn))
            return;
        if(p.tileQuad && (tm * TILE >= p.m || tn * TILE >= p.n))
            return; // a quarter of a partial edge tile that lies outside the matrix
        staggeredStart(p);

        const uint32_t tid  = threadIdx.x;
        const uint32_t lane = tid & 63u;
        const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const uint32_t wm = wave >> 1, wn = wave & 1u;
        const uint32_t ldsBase
            = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) char*)lds));

        uint32_t       gOffA[WB], gOffB[WB], gStepA, gStepB, kByteA, kByteB; // WB direct loads per operand per stage
        uint64_t       gStageA, gStageB;
        const uint32_t validM = p.m - tm * TILE < TILE ? p.m - tm * TILE : TILE;
        const uint32_t validN = p.n - tn * TILE < TILE ? p.n - tn * TILE : TILE;
        laneOffsets8<A_KCONTIG, WB, ES>(tid, p.lda, validM, gOffA, gStepA, gStageA, kByteA);
        laneOffsets8<B_KCONTIG, WB, ES>(tid, p.ldb, validN, gOffB, gStepB, gStageB, kByteB);
        // K need not fill the last stage: its lastBytes (16 .. 128) valid bytes per row are followed by zeros
        // the loads produce themselves (see tailOffset)
        const uint32_t kBytes    = p.k * ES;
        const uint32_t numStages = (kBytes + STAGE_KB - 1u) / STAGE_KB;
        const uint32_t lastBytes = kBytes - (numStages - 1u) * STAGE_KB;
        // (refills past the last stage are issued like all others but with nothing in range: they cost no memory traffic)
        auto validOf = [&](uint32_t stage) { return stage + 1u < numStages ? STAGE_KB : (stage + 1u == numStages ? lastBytes : 0u); };
        const uint32_t dmaDst    = ldsBase + wave * 64u * CHUNK; // + buffer + j * 4 KiB
        auto           uniform64 = [](const char* ptr) {
            const uint64_t v  = reinterpret_cast<uint64_t>(ptr);
            const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
            const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
            return (static_cast<uint64_t>(hi) << 32) | lo;
        };
        const uint64_t gA = uniform64(p.a + (A_KCONTIG ? (uint64_t)tm * TILE * p.lda : (uint64_t)tm * TILE) * ES);
        const uint64_t gB = uniform64(p.b + (B_KCONTIG ? (uint64_t)tn * TILE * p.ldb : (uint64_t)tn * TILE) * ES);
        auto stageAddr = [&](uint64_t panel, uint64_t perStage, uint32_t stage) { // clamped to the last stage
            return panel + (uint64_t)(stage < numStages ? stage : numStages - 1u) * perStage;
        };
        auto issueHalf = [&](bool kContig, uint64_t addr, const uint32_t (&gOff)[WB], uint32_t step, uint32_t kByte, uint32_t ld,
                             uint32_t valid, uint32_t at) {
            const i32x4 rsrc = stageRsrc8(kContig, addr, valid, ld);
#pragma unroll
            for(uint32_t j = 0; j < WB; ++j)
                loadToLds(rsrc, tailOffset(kContig, gOff[j], kByte, valid), j * step, dmaDst + at + j * THREADS * CHUNK);
        };

        uint32_t rdA[8], rdB[8];
        readOffsets8<A_KCONTIG, WB, ES>(wm, lane, rdA);
        readOffsets8<B_KCONTIG, WB, ES>(wn, lane, rdB);

        AccV acc[WB][WB];
#pragma unroll
        for(uint32_t i = 0; i < WB; ++i)
#pragma unroll
            for(uint32_t j = 0; j < WB; ++j)
                acc[i][j] = AccV{0, 0, 0, 0};

        i32x4 fa[2][WB], fb[2][WB];
        // matrix instruction n of a K step: L-shaped shells, as in gemmTiledKernel16
        auto mfmaAt = [&](uint32_t s, uint32_t n) {
            uint32_t d = 0;
            while((d + 1u) * (d + 1u) <= n)
                ++d;
            const uint32_t r = n - d * d;
            const uint32_t i = r <= d ? d : r - d - 1u, j = r <= d ? r : d;
            if constexpr(E == Elem::I8)
                mfma16i8(acc[i][j], fb[s][j], fa[s][i]);
            else if constexpr(E == Elem::F32)
                mfma16f32(acc[i][j], fb[s][j], fa[s][i]);
            else if constexpr(E == Elem::F64)
                mfma16f64(acc[i][j], fb[s][j], fa[s][i]);
            else
                mfma16<E>(acc[i][j], fb[s][j], fa[s][i]);
        };
        // operand block x of K step s: x = 2 i is A block i, x = 2 i + 1 is B block i
        auto readAt = [&](uint32_t aAt, uint32_t bAt, uint32_t s, uint32_t x, uint32_t part) {
            if(x & 1u)
                readBlock8<B_KCONTIG, WB, ES>(lds + bAt, rdB, x >> 1, s, part, fb[s][x >> 1], 0u);
            else
                readBlock8<A_KCONTIG, WB, ES>(lds + aAt, rdA, x >> 1, s, part, fa[s][x >> 1], 0u);
        };

        // One K stage: K step 0 is in registers; step 1 arrives under its matrix instructions; then step 0 of
        // the next stage arrives under the matrix instructions of step 1.  Per four (small wave tile: two) matrix
        // instructions one operand block read (two reads when it is transposed on the way); nothing moves between
        // the pieces.  The direct loads, one at a time between matrix instructions:
        //   large wave tile (SPREAD)  dealt out over the whole stage - B of stage kt + 2 under step 0, into the third
        //       B buffer (free since the barrier of stage kt - 1, not needed before the one of stage kt + 1), A of
        //       stage kt + 2 under step 1, into the A buffer this stage's barrier has freed.  With all of a stage's
        //       loads under step 1 the memory pipeline ran dry during the other half of every stage (int8 8192^3:
        //       0.4145 -> 0.4115 ms; with all-zero operands 0.3230 -> 0.3170).
        //   small wave tile  all under step 1: A of stage kt + 2, then B of stage kt + 3 into the B buffer the barrier
        //       has freed.  Its stages are a quarter as long, and B requested only a stage and a half ahead arrives
        //       late (f16 2048^2 x 8192: 0.0745 ms this way, 0.0770 the other).
        constexpr bool     SPREAD = WB == 8;
        constexpr uint32_t B_AHEAD = SPREAD ? 2u : 3u;
        uint64_t           refillA, refillB; // stage kt + 2 of A, stage kt + B_AHEAD of B (clamped)
        // `full` (compile-time tag): every stage this one requests is a whole stage inside K - the main part of the K
        // loop, whose loads carry no tail select and whose refill pointers always advance
        auto stageBody = [&](auto full, uint32_t kt, uint32_t aCur, uint32_t aNxt, uint32_t bCur, uint32_t bNxt, uint32_t bFree) {
            constexpr bool FULL  = decltype(full)::value;
            const uint32_t vB    = FULL ? STAGE_KB : validOf(kt + B_AHEAD);
            const i32x4    rsrcB = stageRsrc8(B_KCONTIG, refillB, vB, p.ldb);
            if(FULL || kt + B_AHEAD + 1u < numStages)
                refillB += gStageB;
            auto offA = [&](uint32_t j, uint32_t valid) { return FULL ? gOffA[j] : tailOffset(A_KCONTIG, gOffA[j], kByteA, valid); };
            auto offB = [&](uint32_t j, uint32_t valid) { return FULL ? gOffB[j] : tailOffset(B_KCONTIG, gOffB[j], kByteB, valid); };
#pragma unroll
            for(uint32_t x = 0; x < XS; ++x)
#pragma unroll
                for(uint32_t q = 0; q < QS; ++q)
                {
                    mfmaAt(0, QS * x + q);
                    if(q < 2u)
                        readAt(aCur, bCur, 1, x, q);
                    if constexpr(SPREAD)
                        if(q == LOAD_Q && (x & 1u))
                            loadToLds(rsrcB, offB(x >> 1, vB), (x >> 1) * gStepB, dmaDst + bFree + (x >> 1) * THREADS * CHUNK);
                    __builtin_amdgcn_sched_barrier(0);
                }
            waitVmcnt<WB>(); // this wave's part of stage kt + 1 has landed (the youngest WB loads are B of kt + 2)
            ldsBarrier();
            const uint32_t vA    = FULL ? STAGE_KB : validOf(kt + 2u);
            const i32x4    rsrcA = stageRsrc8(A_KCONTIG, refillA, vA, p.lda);
            if(FULL || kt + 3u < numStages)
                refillA += gStageA;
#pragma unroll
            for(uint32_t x = 0; x < XS; ++x)
#pragma unroll
                for(uint32_t q = 0; q < QS; ++q)
                {
                    mfmaAt(1, QS * x + q);
                    if(q < 2u)
                        readAt(aNxt, bNxt, 0, x, q);
                    if constexpr(SPREAD)
                    {
                        if(q == LOAD_Q && (x & 1u))
                            loadToLds(rsrcA, offA(x >> 1, vA), (x >> 1) * gStepA, dmaDst + aCur + (x >> 1) * THREADS * CHUNK);
                    }
                    else if(q == LOAD_Q)
                    {
                        if(x < WB)
                            loadToLds(rsrcA, offA(x, vA), x * gStepA, dmaDst + aCur + x * THREADS * CHUNK);
                        else
                            loadToLds(rsrcB, offB(x - WB, vB), (x - WB) * gStepB, dmaDst + bCur + (x - WB) * THREADS * CHUNK);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
        };

        // prologue: stages 0 and 1 (and, where B runs three stages ahead, B of stage 2) requested in the order the
        // loop keeps; stage 0 published
        if constexpr(SPREAD)
        {
            issueHalf(B_KCONTIG, stageAddr(gB, gStageB, 0u), gOffB, gStepB, kByteB, p.ldb, validOf(0u), B_AT[0]);
            issueHalf(A_KCONTIG, stageAddr(gA, gStageA, 0u), gOffA, gStepA, kByteA, p.lda, validOf(0u), A_AT[0]);
            issueHalf(B_KCONTIG, stageAddr(gB, gStageB, 1u), gOffB, gStepB, kByteB, p.ldb, validOf(1u), B_AT[1]);
            issueHalf(A_KCONTIG, stageAddr(gA, gStageA, 1u), gOffA, gStepA, kByteA, p.lda, validOf(1u), A_AT[1]);
            waitVmcnt<2u * WB>();
        }
        else
        {
            issueHalf(A_KCONTIG, stageAddr(gA, gStageA, 0u), gOffA, gStepA, kByteA, p.lda, validOf(0u), A_AT[0]);
            issueHalf(B_KCONTIG, stageAddr(gB, gStageB, 0u), gOffB, gStepB, kByteB, p.ldb, validOf(0u), B_AT[0]);
            issueHalf(A_KCONTIG, stageAddr(gA, gStageA, 1u), gOffA, gStepA, kByteA, p.lda, validOf(1u), A_AT[1]);
            issueHalf(B_KCONTIG, stageAddr(gB, gStageB, 1u), gOffB, gStepB, kByteB, p.ldb, validOf(1u), B_AT[1]);
            issueHalf(B_KCONTIG, stageAddr(gB, gStageB, 2u), gOffB, gStepB, kByteB, p.ldb, validOf(2u), B_AT[2]);
            waitVmcnt<3u * WB>();
        }
        refillA = stageAddr(gA, gStageA, 2u), refillB = stageAddr(gB, gStageB, B_AHEAD);
        ldsBarrier();
        R355_STAMP(1);
#pragma unroll
        for(uint32_t x = 0; x < XS; ++x)
        {
            readAt(A_AT[0], B_AT[0], 0, x, 0);
            readAt(A_AT[0], B_AT[0], 0, x, 1);
        }

        // six stages per trip bring every buffer back to its role; single-exit loops, then the remainder.  The main part
        // runs the trips whose requests (up to stage kt + 5 + B_AHEAD) all are whole stages inside K without the tail
        // handling; the trips around the end of K and the remainder carry it.
        // (Only a K-contiguous operand has a select to lose: with none, the main part is empty and compiles away.)
        const uint32_t     wholeStages = (A_KCONTIG || B_KCONTIG) ? kBytes / STAGE_KB : 0u;
        constexpr uint32_t REACH       = 5u + B_AHEAD;
        const uint32_t     mainTrips   = wholeStages > REACH ? (wholeStages - REACH + 5u) / 6u : 0u;
        using Main = std::true_type;
        using Tail = std::false_type;
        uint32_t kt = 0;
        for(uint32_t trips = mainTrips; trips > 0; --trips, kt += 6u)
        {
            stageBody(Main{}, kt, A_AT[0], A_AT[1], B_AT[0], B_AT[1], B_AT[2]);
            stageBody(Main{}, kt + 1u, A_AT[1], A_AT[0], B_AT[1], B_AT[2], B_AT[0]);
            stageBody(Main{}, kt + 2u, A_AT[0], A_AT[1], B_AT[2], B_AT[0], B_AT[1]);
            stageBody(Main{}, kt + 3u, A_AT[1], A_AT[0], B_AT[0], B_AT[1], B_AT[2]);
            stageBody(Main{}, kt + 4u, A_AT[0], A_AT[1], B_AT[1], B_AT[2], B_AT[0]);
            stageBody(Main{}, kt + 5u, A_AT[1], A_AT[0], B_AT[2], B_AT[0], B_AT[1]);
        }
        for(uint32_t trips = numStages / 6u - mainTrips; trips > 0; --trips, kt += 6u)
        {
            stageBody(Tail{}, kt, A_AT[0], A_AT[1], B_AT[0], B_AT[1], B_AT[2]);
            stageBody(Tail{}, kt + 1u, A_AT[1], A_AT[0], B_AT[1], B_AT[2], B_AT[0]);
            stageBody(Tail{}, kt + 2u, A_AT[0], A_AT[1], B_AT[2], B_AT[0], B_AT[1]);
            stageBody(Tail{}, kt + 3u, A_AT[1], A_AT[0], B_AT[0], B_AT[1], B_AT[2]);
            stageBody(Tail{}, kt + 4u, A_AT[0], A_AT[1], B_AT[1], B_AT[2], B_AT[0]);
            stageBody(Tail{}, kt + 5u, A_AT[1], A_AT[0], B_AT[2], B_AT[0], B_AT[1]);
        }
        const uint32_t rem = numStages - kt;
        if(rem > 0u)
        {
            stageBody(Tail{}, kt, A_AT[0], A_AT[1], B_AT[0], B_AT[1], B_AT[2]);
            if(rem > 1u)
            {
                stageBody(Tail{}, kt + 1u, A_AT[1], A_AT[0], B_AT[1], B_AT[2], B_AT[0]);
                if(rem > 2u)
                {
                    stageBody(Tail{}, kt + 2u, A_AT[0], A_AT[1], B_AT[2], B_AT[0], B_AT[1]);
                    if(rem > 3u)
                    {
                        stageBody(Tail{}, kt + 3u, A_AT[1], A_AT[0], B_AT[0], B_AT[1], B_AT[2]);
                        if(rem > 4u)
                            stageBody(Tail{}, kt + 4u, A_AT[0], A_AT[1], B_AT[1], B_AT[2], B_AT[0]);
                    }
                }
            }
        }

        R355_STAMP(2);
        // the loads past the last stage (zeros) are still landing in buffers the epilogue reuses, and the
        // last matrix instructions are still in the pipeline (the compiler does not know either)
        asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
        waitVmcnt<0>();
        ldsBarrier();
        storeTile16<AccV, OutT, WB, WB>(acc, p, tm * TILE + wm * WT, tn * TILE + wn * WT, lane, lds + wave * (WB * 4096u));
        R355_STAMP_END();
    }

    // ------------------------------------------------------------------------------------------
    // int8, the 256 x 256 macro tile on EIGHT waves: two waves per SIMD, 2 x 4 waves with wave tiles of 128 x 64 (8 x 4
    // accumulator blocks = 128 registers, so two waves fit a SIMD's register file).  With one wave per SIMD every LDS read
    // or direct load that its unit cannot take at once holds up the matrix instruction behind it (a wave issues in
    // order); here the SIMD's other wave can issue meanwhile.  The price: every wave reads 12 operand blocks per 32 matrix
    // instructions instead of 16 per 64 (1.5 x the LDS read volume).  Same five LDS buffers, same K-step structure and
    // the same storage swizzles as gemmTiled5; 512 threads move a 32 KiB operand tile in 4 loads each.
    constexpr uint32_t THREADS_WIDE = 512;

    template <bool KCONTIG>
    __device__ __forceinline__ void laneOffsetsWide(uint32_t tid, uint32_t ld, uint32_t valid, uint32_t (&off)[4], uint32_t& step,
                                                    uint64_t& stage, uint32_t& kByte)
    {
        kByte = 0u;
        if constexpr(KCONTIG)
        {
            const uint32_t r = tid >> 3, slot = tid & 7u; // chunk j * 512 + tid: row 64 j + r (the swizzle does not change with j)
            kByte            = (slot ^ swzK8(r)) * CHUNK;
#pragma unroll
            for(uint32_t j = 0; j < 4; ++j)
            {
                const uint32_t row = r + 64u * j < valid ? r + 64u * j : valid - 1u;
                off[j]             = row * ld + kByte;
            }
            step = 0u, stage = STAGE_KB;
        }
        else
        {
            const uint32_t r = tid >> 4, slot = tid & 15u; // k-row 32 j + r: bits 0 .. 2 and 4 of it, which the swizzle uses, are r's
#pragma unroll
            for(uint32_t j = 0; j < 4; ++j)
            {
                const uint32_t c = slot ^ swzMN8<8>(32u * j + r);
                off[j]           = r * ld + (c * CHUNK < valid ? c : 0u) * CHUNK;
            }
            step = 32u * ld, stage = (uint64_t)STAGE_KB * ld;
        }
    }

    template <typename OutT, bool A_KCONTIG, bool B_KCONTIG>
    __device__ __forceinline__ void gemmTiledI8Wide(const Params& p)
    {
        constexpr uint32_t WBM = 8, WBN = 4, TILE = 256, OPER = TILE * STAGE_KB; // wave tile 128 x 64; 32 KiB per operand and stage
        constexpr uint32_t NL = OPER / CHUNK / THREADS_WIDE; // 4 direct loads per operand, stage and thread
        constexpr uint32_t NM = WBM * WBN; // 32 matrix instructions per K step
        constexpr uint32_t A_AT[2] = {0u, OPER};
        constexpr uint32_t B_AT[3] = {2u * OPER, 3u * OPER, 4u * OPER};
        __shared__ __attribute__((aligned(1024))) char lds[5u * OPER];

        uint32_t tm, tn;
        if(!r355::tileCoordRange(blockIdx.x, p.tilesM, p.tilesN, p.tileFirst, p.tileCount, false, tm, tn))
            return;
        staggeredStart(p);
        const uint32_t tid  = threadIdx.x;
        const uint32_t lane = tid & 63u;
        const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const uint32_t wm = wave >> 2, wn = wave & 3u;
        const uint32_t t = lane & 15u, g = lane >> 4;
        const uint32_t ldsBase
            = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) char*)lds));

        uint32_t       gOffA[NL], gOffB[NL], gStepA, gStepB, kByteA, kByteB;
        uint64_t       gStageA, gStageB;
        const uint32_t validM = p.m - tm * TILE < TILE ? p.m - tm * TILE : TILE;
        const uint32_t validN = p.n - tn * TILE < TILE ? p.n - tn * TILE : TILE;
        laneOffsetsWide<A_KCONTIG>(tid, p.lda, validM, gOffA, gStepA, gStageA, kByteA);
        laneOffsetsWide<B_KCONTIG>(tid, p.ldb, validN, gOffB, gStepB, gStageB, kByteB);
        const uint32_t numStages = (p.k + STAGE_KB - 1u) / STAGE_KB;
        const uint32_t lastBytes = p.k - (numStages - 1u) * STAGE_KB;
        auto validOf = [&](uint32_t stage) { return stage + 1u < numStages ? STAGE_KB : (stage + 1u == numStages ? lastBytes : 0u); };
        const uint32_t dmaDst = ldsBase + wave * 64u * CHUNK; // + buffer + j * 8 KiB
        const uint64_t gA = r355::uniformAddress(p.a + (A_KCONTIG ? (uint64_t)tm * TILE * p.lda : (uint64_t)tm * TILE));
        const uint64_t gB = r355::uniformAddress(p.b + (B_KCONTIG ? (uint64_t)tn * TILE * p.ldb : (uint64_t)tn * TILE));
        auto stageAddr = [&](uint64_t panel, uint64_t perStage, uint32_t stage) { // clamped to the last stage
            return panel + (uint64_t)(stage < numStages ? stage : numStages - 1u) * perStage;
        };
        auto issueHalf = [&](bool kContig, uint64_t addr, const uint32_t (&gOff)[NL], uint32_t step, uint32_t kByte, uint32_t ld,
                             uint32_t valid, uint32_t at) {
            const i32x4 rsrc = stageRsrc8(kContig, addr, valid, ld);
#pragma unroll
            for(uint32_t j = 0; j < NL; ++j)
                loadToLds(rsrc, tailOffset(kContig, gOff[j], kByte, valid), j * step, dmaDst + at + j * THREADS_WIDE * CHUNK);
        };

        // LDS -> registers: K-contiguous rd[q] is 64-byte K step q of block 0 (block i 16 rows further); M/N-contiguous rd[i]
        // is block i (16-byte chunk first + i of the 256-byte k-rows), the first 8 k-rows of the lane's 16 of K step 0
        uint32_t rdA[8], rdB[8];
        auto readOffsets = [&](bool kContig, uint32_t firstBlock, uint32_t blocks, uint32_t (&rd)[8]) {
#pragma unroll
            for(uint32_t i = 0; i < 8; ++i)
                rd[i] = 0u;
            if(kContig)
            {
                const uint32_t r = firstBlock * 16u + t;
                rd[0]            = r * STAGE_KB + ((g ^ swzK8(r)) * CHUNK);
                rd[1]            = r * STAGE_KB + (((4u + g) ^ swzK8(r)) * CHUNK);
            }
            else
            {
                const uint32_t kr = 16u * g + (t >> 1);
#pragma unroll
                for(uint32_t i = 0; i < 8; ++i)
                    if(i < blocks)
                        rd[i] = kr * 256u + (((firstBlock + i) ^ swzMN8<8>(kr)) * CHUNK) + (t & 1u) * 8u;
            }
        };
        readOffsets(A_KCONTIG, wm * WBM, WBM, rdA);
        readOffsets(B_KCONTIG, wn * WBN, WBN, rdB);

        i32x4v acc[WBM][WBN];
#pragma unroll
        for(uint32_t i = 0; i < WBM; ++i)
#pragma unroll
            for(uint32_t j = 0; j < WBN; ++j)
                acc[i][j] = i32x4v{0, 0, 0, 0};

        i32x4 fa[2][WBM], fb[2][WBN];
        // Matrix instruction n (0 .. 31) of a K step: the 4 x 4 corner in L-shaped shells, then block rows 4 .. 7; the
        // operand blocks are read in the order they are first needed: A0 B0 A1 B1 A2 B2 A3 B3 A4 A5 A6 A7.
        auto mfmaAt = [&](uint32_t s, uint32_t n) {
            uint32_t i, j;
            if(n < WBN * WBN)
            {
                uint32_t d = 0;
                while((d + 1u) * (d + 1u) <= n)
                    ++d;
                const uint32_t r = n - d * d;
                i = r <= d ? d : r - d - 1u, j = r <= d ? r : d;
            }
            else
                i = n / WBN, j = n % WBN;
            mfma16i8(acc[i][j], fb[s][j], fa[s][i]);
        };
        // read piece r of a K step: the blocks in the order above, one piece each when K-contiguous, two (the halves
        // of a transposing read pair) otherwise; pieces are dealt out evenly over the 32 slots of the previous K step
        constexpr uint32_t PA = A_KCONTIG ? 1u : 2u, PB = B_KCONTIG ? 1u : 2u;
        constexpr uint32_t NR = WBM * PA + WBN * PB;
        auto readPiece = [&](uint32_t aAt, uint32_t bAt, uint32_t s, uint32_t r) {
            // pieces of blocks 0 .. 3 alternate A, B; then A's blocks 4 .. 7
            uint32_t left = r;
#pragma unroll
            for(uint32_t x = 0; x < WBM + WBN; ++x)
            {
                const bool     isB = x < 2u * WBN && (x & 1u);
                const uint32_t blk = x < 2u * WBN ? x >> 1 : x - WBN, parts = isB ? PB : PA;
                if(left < parts)
                {
                    if(isB)
                        readBlock8<B_KCONTIG, 8>(lds + bAt, rdB, blk, s, left, fb[s][blk], 0u);
                    else
                        readBlock8<A_KCONTIG, 8>(lds + aAt, rdA, blk, s, left, fa[s][blk], 0u);
                    return;
                }
                left -= parts;
            }
        };
        auto readSlot = [&](uint32_t aAt, uint32_t bAt, uint32_t s, uint32_t n) {
#pragma unroll
            for(uint32_t r = (n * NR + NM - 1u) / NM; r < ((n + 1u) * NR + NM - 1u) / NM; ++r)
                readPiece(aAt, bAt, s, r);
        };

        uint64_t refillA, refillB; // stage kt + 2 of A and of B (clamped)
        auto stageBody = [&](auto full, uint32_t kt, uint32_t aCur, uint32_t aNxt, uint32_t bCur, uint32_t bNxt, uint32_t bFree) {
            constexpr bool FULL  = decltype(full)::value;
            const uint32_t vB    = FULL ? STAGE_KB : validOf(kt + 2u);
            const i32x4    rsrcB = stageRsrc8(B_KCONTIG, refillB, vB, p.ldb);
            if(FULL || kt + 3u < numStages)
                refillB += gStageB;
#pragma unroll
            for(uint32_t n = 0; n < NM; ++n)
            {
                mfmaAt(0, n);
                readSlot(aCur, bCur, 1, n);
                if(n % 8u == 3u) // B of stage kt + 2 into the third B buffer
                    loadToLds(rsrcB, FULL ? gOffB[n / 8u] : tailOffset(B_KCONTIG, gOffB[n / 8u], kByteB, vB), (n / 8u) * gStepB,
                              dmaDst + bFree + (n / 8u) * THREADS_WIDE * CHUNK);
                __builtin_amdgcn_sched_barrier(0);
            }
            waitVmcnt<NL>(); // this wave's part of stage kt + 1 has landed (the youngest NL loads are B of kt + 2)
            ldsBarrier();
            const uint32_t vA    = FULL ? STAGE_KB : validOf(kt + 2u);
            const i32x4    rsrcA = stageRsrc8(A_KCONTIG, refillA, vA, p.lda);
            if(FULL || kt + 3u < numStages)
                refillA += gStageA;
#pragma unroll
            for(uint32_t n = 0; n < NM; ++n)
            {
                mfmaAt(1, n);
                readSlot(aNxt, bNxt, 0, n);
                if(n % 8u == 3u) // A of stage kt + 2 into the A buffer this stage's barrier has freed
                    loadToLds(rsrcA, FULL ? gOffA[n / 8u] : tailOffset(A_KCONTIG, gOffA[n / 8u], kByteA, vA), (n / 8u) * gStepA,
                              dmaDst + aCur + (n / 8u) * THREADS_WIDE * CHUNK);
                __builtin_amdgcn_sched_barrier(0);
            }
        };

        issueHalf(B_KCONTIG, stageAddr(gB, gStageB, 0u), gOffB, gStepB, kByteB, p.ldb, validOf(0u), B_AT[0]);
        issueHalf(A_KCONTIG, stageAddr(gA, gStageA, 0u), gOffA, gStepA, kByteA, p.lda, validOf(0u), A_AT[0]);
        issueHalf(B_KCONTIG, stageAddr(gB, gStageB, 1u), gOffB, gStepB, kByteB, p.ldb, validOf(1u), B_AT[1]);
        issueHalf(A_KCONTIG, stageAddr(gA, gStageA, 1u), gOffA, gStepA, kByteA, p.lda, validOf(1u), A_AT[1]);
        waitVmcnt<2u * NL>();
        refillA = stageAddr(gA, gStageA, 2u), refillB = stageAddr(gB, gStageB, 2u);
        ldsBarrier();
#pragma unroll
        for(uint32_t r = 0; r < NR; ++r)
            readPiece(A_AT[0], B_AT[0], 0, r);

        const uint32_t wholeStages = (A_KCONTIG || B_KCONTIG) ? p.k / STAGE_KB : 0u;
        const uint32_t mainTrips   = wholeStages > 7u ? (wholeStages - 7u + 5u) / 6u : 0u;
        using Main = std::true_type;
        using Tail = std::false_type;
        uint32_t kt = 0;
        for(uint32_t trips = mainTrips; trips > 0; --trips, kt += 6u)
        {
            stageBody(Main{}, kt, A_AT[0], A_AT[1], B_AT[0], B_AT[1], B_AT[2]);
            stageBody(Main{}, kt + 1u, A_AT[1], A_AT[0], B_AT[1], B_AT[2], B_AT[0]);
            stageBody(Main{}, kt + 2u, A_AT[0], A_AT[1], B_AT[2], B_AT[0], B_AT[1]);
            stageBody(Main{}, kt + 3u, A_AT[1], A_AT[0], B_AT[0], B_AT[1], B_AT[2]);
            stageBody(Main{}, kt + 4u, A_AT[0], A_AT[1], B_AT[1], B_AT[2], B_AT[0]);
            stageBody(Main{}, kt + 5u, A_AT[1], A_AT[0], B_AT[2], B_AT[0], B_AT[1]);
        }
        for(uint32_t trips = numStages / 6u - mainTrips; trips > 0; --trips, kt += 6u)
        {
            stageBody(Tail{}, kt, A_AT[0], A_AT[1], B_AT[0], B_AT[1], B_AT[2]);
            stageBody(Tail{}, kt + 1u, A_AT[1], A_AT[0], B_AT[1], B_AT[2], B_AT[0]);
            stageBody(Tail{}, kt + 2u, A_AT[0], A_AT[1], B_AT[2], B_AT[0], B_AT[1]);
            stageBody(Tail{}, kt + 3u, A_AT[1], A_AT[0], B_AT[0], B_AT[1], B_AT[2]);
            stageBody(Tail{}, kt + 4u, A_AT[0], A_AT[1], B_AT[1], B_AT[2], B_AT[0]);
            stageBody(Tail{}, kt + 5u, A_AT[1], A_AT[0], B_AT[2], B_AT[0], B_AT[1]);
        }
        const uint32_t rem = numStages - kt;
        if(rem > 0u)
        {
            stageBody(Tail{}, kt, A_AT[0], A_AT[1], B_AT[0], B_AT[1], B_AT[2]);
            if(rem > 1u)
            {
                stageBody(Tail{}, kt + 1u, A_AT[1], A_AT[0], B_AT[1], B_AT[2], B_AT[0]);
                if(rem > 2u)
                {
                    stageBody(Tail{}, kt + 2u, A_AT[0], A_AT[1], B_AT[2], B_AT[0], B_AT[1]);
                    if(rem > 3u)
                    {
                        stageBody(Tail{}, kt + 3u, A_AT[1], A_AT[0], B_AT[0], B_AT[1], B_AT[2]);
                        if(rem > 4u)
                            stageBody(Tail{}, kt + 4u, A_AT[0], A_AT[1], B_AT[1], B_AT[2], B_AT[0]);
                    }
                }
            }
        }
        asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
        waitVmcnt<0>();
        ldsBarrier();
        storeTile16<i32x4v, OutT, WBM, WBN, 16384u>(acc, p, tm * TILE + wm * (16u * WBM), tn * TILE + wn * (16u * WBN), lane,
                                                    lds + wave * 16384u);
    }

    template <typename OutT, bool A_KCONTIG, bool B_KCONTIG>
    __global__ void __launch_bounds__(THREADS_WIDE) __attribute__((amdgpu_waves_per_eu(2, 2))) gemmTiledKernelI8Wide(Params p)
    {
        gemmTiledI8Wide<OutT, A_KCONTIG, B_KCONTIG>(p);
    }

    template <typename OutT, bool A_KCONTIG, bool B_KCONTIG>
    __global__ void __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(1, 1))) gemmTiledKernelI8(Params p)
    {
        gemmTiled5<Elem::I8, OutT, A_KCONTIG, B_KCONTIG, 8>(p);
    }
    template <typename OutT, bool A_KCONTIG, bool B_KCONTIG>
    __global__ void __launch_bounds__(THREADS) gemmTiledKernelI8Small(Params p)
    {
        gemmTiled5<Elem::I8, OutT, A_KCONTIG, B_KCONTIG, 4>(p);
    }
    template <bool A_KCONTIG, bool B_KCONTIG>
    __global__ void __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(1, 1))) gemmTiledKernelF32(Params p)
    {
        gemmTiled5<Elem::F32, float, A_KCONTIG, B_KCONTIG, 8>(p);
    }
    template <bool A_KCONTIG, bool B_KCONTIG>
    __global__ void __launch_bounds__(THREADS) gemmTiledKernelF32Small(Params p)
    {
        gemmTiled5<Elem::F32, float, A_KCONTIG, B_KCONTIG, 4>(p);
    }
    template <bool A_KCONTIG, bool B_KCONTIG>
    __global__ void __launch_bounds__(THREADS) gemmTiledKernelF64Small(Params p)
    {
        gemmTiled5<Elem::F64, double, A_KCONTIG, B_KCONTIG, 4>(p);
    }
    // The 128 x 128 tile of f16 / bf16 runs the five-buffer body as well: with a stage lasting a quarter as
    // long, the two-buffer scheme of gemmTiled16 keeps too little in flight (2048^3 f16: 710 TFLOP/s against 887
    // here).  For the 256 x 256 tile the two-buffer kernel stays 1-2 % ahead (it is power-bound, not latency-bound).
    template <Elem E, typename OutT, bool A_KCONTIG, bool B_KCONTIG>
    __global__ void __launch_bounds__(THREADS) gemmTiledKernel16Small(Params p)
    {
        gemmTiled5<E, OutT, A_KCONTIG, B_KCONTIG, 4>(p);
    }
    // The 256 x 256 tile of f16 / bf16 on the five-buffer body: loads two to three stages ahead instead of one.  While the
    // operands stay in the 256 MiB memory-side cache the two-buffer kernel is 1 - 2.6 % ahead; once A and B together
    // exceed it, panels are re-fetched from HBM and one stage of lookahead no longer covers the latency
    // (8192^2 x 16384 TN: 1268 against 1435 TFLOP/s here; 8192 x 12288 x 8192 NN: 1317 against 1474; this body within
    // 1430 - 1490 over every size and orientation tried).
    template <Elem E, typename OutT, bool A_KCONTIG, bool B_KCONTIG>
    __global__ void __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(1, 1))) gemmTiledKernel16Deep(Params p)
    {
        gemmTiled5<E, OutT, A_KCONTIG, B_KCONTIG, 8>(p);
    }

    // ------------------------------------------------------------------------------------------
    // fp8 e4m3 on v_mfma_f32_16x16x128_f8f6f4.  One instruction spans the whole 128-byte K stage
    // (32 bytes per lane: K bytes 16 (lane / 16) .. + 15 of each 64-byte half, a K permutation shared by
    // A and B), so a stage cannot be split along K.  It is split into quadrants of the wave tile instead:
    //     Q1 = A[0..3] x B[0..3]   Q2 = A[0..3] x B[4..7]   Q3 = A[4..7] x B[4..7]   Q4 = A[4..7] x B[0..3]
    // Consecutive quadrants share one operand group (4 blocks, 32 registers), so each quadrant's 16
    // matrix instructions hide the LDS reads (8, or 16 transposing ones) of the one group the next
    // quadrant needs:
    //     under Q1: B[4..7] of this stage       under Q3: A[0..3] of the next stage
    //     under Q2: A[4..7] of this stage       under Q4: B[0..3] of the next stage
    // After Q2 the stage's buffers are no longer read: barrier, then the refills are issued under Q3
    // (A) and Q4 (B).  Four register groups suffice; the two B groups swap roles every stage.
    using i32x8 = int __attribute__((ext_vector_type(8)));
    template <bool E5M2>
    __device__ __forceinline__ void mfma16f8(f32x4& acc, const i32x8& x, const i32x8& y)
    {
        // cbsz / blgp give the formats of the two operands: 0 = e4m3, 1 = e5m2; the unscaled form multiplies by 2^0
        if constexpr(E5M2)
            asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0 cbsz:1 blgp:1" : "+a"(acc) : "v"(x), "v"(y));
        else
            asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+a"(acc) : "v"(x), "v"(y));
    }

    template <bool E5M2, bool A_KCONTIG, bool B_KCONTIG, uint32_t WB>
    __device__ __forceinline__ void gemmTiledF8(const Params& whole)
    {
        static_assert(WB == 8 || WB == 4, "wave tile of 8 x 8 or 4 x 4 blocks");
        R355_STAMP(0);
        R355_STAMP_ID();
        const Params p = splitShare<1u>(whole, A_KCONTIG ? (uint64_t)STAGE_KB : (uint64_t)STAGE_KB * whole.lda,
                                        B_KCONTIG ? (uint64_t)STAGE_KB : (uint64_t)STAGE_KB * whole.ldb);
        constexpr uint32_t TILE = 32u * WB, WT = 16u * WB; // macro tile and wave tile edge
        constexpr uint32_t OPER = TILE * STAGE_KB; // bytes of one operand per stage: 32 or 16 KiB
        constexpr uint32_t H = WB / 2u, NQ = H * H; // blocks per operand group, matrix instructions per quadrant
        constexpr uint32_t A_AT[2] = {0u, OPER};
        constexpr uint32_t B_AT[3] = {2u * OPER, 3u * OPER, 4u * OPER};
        __shared__ __attribute__((aligned(1024))) char lds[5u * OPER];

        uint32_t tm, tn;
        if(!r355::tileCoordRange(blockIdx.x, p.tilesM, p.tilesN, p.tileFirst, p.tileCount, p.tileQuad != 0u, tm, tn))
            return;
        if(p.tileQuad && (tm * TILE >= p.m || tn * TILE >= p.n))
            return; // a quarter of a partial edge tile that lies outside the matrix
        staggeredStart(p);

        const uint32_t tid  = threadIdx.x;
        const uint32_t lane = tid & 63u;
        const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const uint32_t wm = wave >> 1, wn = wave & 1u;
        const uint32_t ldsBase
            = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) char*)lds));

        uint32_t       gOffA[WB], gOffB[WB], gStepA, gStepB, kByteA, kByteB; // WB direct loads per operand per stage
        uint64_t       gStageA, gStageB;
        const uint32_t validM = p.m - tm * TILE < TILE ? p.m - tm * TILE : TILE;
        const uint32_t validN = p.n - tn * TILE < TILE ? p.n - tn * TILE : TILE;
        laneOffsets8<A_KCONTIG, WB>(tid, p.lda, validM, gOffA, gStepA, gStageA, kByteA);
        laneOffsets8<B_KCONTIG, WB>(tid, p.ldb, validN, gOffB, gStepB, gStageB, kByteB);
        // K need not fill the last stage: its lastBytes (16 .. 128) valid bytes per row are followed by zeros
        // the loads produce themselves (see tailOffset)
        const uint32_t numStages = (p.k + STAGE_KB - 1u) / STAGE_KB;
        const uint32_t lastBytes = p.k - (numStages - 1u) * STAGE_KB;
        // (refills past the last stage are issued like all others but with nothing in range: they cost no memory traffic)
        auto validOf = [&](uint32_t stage) { return stage + 1u < numStages ? STAGE_KB : (stage + 1u == numStages ? lastBytes : 0u); };
        const uint32_t dmaDst    = ldsBase + wave * 64u * CHUNK;
        auto           uniform64 = [](const char* ptr) {
            const uint64_t v  = reinterpret_cast<uint64_t>(ptr);
            const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
            const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
            return (static_cast<uint64_t>(hi) << 32) | lo;
        };
        const uint64_t gA = uniform64(p.a + (A_KCONTIG ? (uint64_t)tm * TILE * p.lda : (uint64_t)tm * TILE));
        const uint64_t gB = uniform64(p.b + (B_KCONTIG ? (uint64_t)tn * TILE * p.ldb : (uint64_t)tn * TILE));
        auto stageAddr = [&](uint64_t panel, uint64_t perStage, uint32_t stage) {
            return panel + (uint64_t)(stage < numStages ? stage : numStages - 1u) * perStage;
        };
        auto issueHalf = [&](bool kContig, uint64_t addr, const uint32_t (&gOff)[WB], uint32_t step, uint32_t kByte, uint32_t ld,
                             uint32_t valid, uint32_t at) {
            const i32x4 rsrc = stageRsrc8(kContig, addr, valid, ld);
#pragma unroll
            for(uint32_t j = 0; j < WB; ++j)
                loadToLds(rsrc, tailOffset(kContig, gOff[j], kByte, valid), j * step, dmaDst + at + j * THREADS * CHUNK);
        };

        uint32_t rdA[8], rdB[8];
        readOffsets8<A_KCONTIG, WB>(wm, lane, rdA);
        readOffsets8<B_KCONTIG, WB>(wn, lane, rdB);
        // An operand group (blocks H half .. + H - 1) arrives in 2 H pieces of 16 bytes (K-contiguous:
        // piece r is block r / 2, 64-byte half r % 2) or 4 H transposed pieces of 8 bytes (block r / 4,
        // half (r / 2) % 2, part r % 2), dealt out evenly over the NQ slots of a quadrant.
        auto readSlotA = [&](i32x8 (&grp)[H], uint32_t at, uint32_t half, uint32_t n) {
            constexpr uint32_t P = A_KCONTIG ? 2u * H : 4u * H;
#pragma unroll
            for(uint32_t r = (n * P + NQ - 1u) / NQ; r < ((n + 1u) * P + NQ - 1u) / NQ; ++r)
            {
                const uint32_t b = A_KCONTIG ? r >> 1 : r >> 2, kh = A_KCONTIG ? r & 1u : (r >> 1) & 1u, part = A_KCONTIG ? 0u : r & 1u;
                readBlock8<A_KCONTIG, WB>(lds + at, rdA, H * half + b, kh, part, grp[b], 4u * kh);
            }
        };
        auto readSlotB = [&](i32x8 (&grp)[H], uint32_t at, uint32_t half, uint32_t n) {
            constexpr uint32_t P = B_KCONTIG ? 2u * H : 4u * H;
#pragma unroll
            for(uint32_t r = (n * P + NQ - 1u) / NQ; r < ((n + 1u) * P + NQ - 1u) / NQ; ++r)
            {
                const uint32_t b = B_KCONTIG ? r >> 1 : r >> 2, kh = B_KCONTIG ? r & 1u : (r >> 1) & 1u, part = B_KCONTIG ? 0u : r & 1u;
                readBlock8<B_KCONTIG, WB>(lds + at, rdB, H * half + b, kh, part, grp[b], 4u * kh);
            }
        };
        // direct load j of an operand goes out in slot n when [n WB / NQ, (n + 1) WB / NQ) contains j
        // (`full`, a compile-time tag: the stage is a whole one inside K, no lane has a chunk beyond K)
        auto loadSlot = [&](auto full, bool kContig, const i32x4& rsrc, const uint32_t (&gOff)[WB], uint32_t step, uint32_t kByte,
                            uint32_t valid, uint32_t at, uint32_t n) {
#pragma unroll
            for(uint32_t j = n * WB / NQ; j < (n + 1u) * WB / NQ; ++j)
                loadToLds(rsrc, decltype(full)::value ? gOff[j] : tailOffset(kContig, gOff[j], kByte, valid), j * step,
                          dmaDst + at + j * THREADS * CHUNK);
        };

        f32x4 acc[WB][WB];
#pragma unroll
        for(uint32_t i = 0; i < WB; ++i)
#pragma unroll
            for(uint32_t j = 0; j < WB; ++j)
                acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

        i32x8 aLo[H], aHi[H], bX[H], bY[H]; // bX / bY alternate as the low / high half of B's blocks

        uint64_t refillA, refillB; // stage kt + 2 of A, stage kt + 3 of B (clamped)
        // `full` (compile-time tag): the stages this one requests (kt + 2 of A, kt + 3 of B) are whole stages inside K -
        // the main part of the K loop, without tail selects and with refill pointers that always advance
        auto stageBody = [&](auto full, uint32_t kt, uint32_t aCur, uint32_t aNxt, uint32_t bCur, uint32_t bNxt, i32x8 (&bLo)[H],
                             i32x8 (&bHi)[H]) {
            constexpr bool FULL = decltype(full)::value;
            // Q1: A low x B low; B high arrives
#pragma unroll
            for(uint32_t n = 0; n < NQ; ++n)
            {
                mfma16f8<E5M2>(acc[n % H][n / H], bLo[n / H], aLo[n % H]);
                readSlotB(bHi, bCur, 1, n);
                __builtin_amdgcn_sched_barrier(0);
            }
            // Q2: A low x B high (column by column, in the order B arrived); A high arrives
#pragma unroll
            for(uint32_t n = 0; n < NQ; ++n)
            {
                mfma16f8<E5M2>(acc[n % H][H + n / H], bHi[n / H], aLo[n % H]);
                readSlotA(aHi, aCur, 1, n);
                __builtin_amdgcn_sched_barrier(0);
            }
            waitVmcnt<WB>(); // this wave's part of stage kt + 1 has landed (the youngest WB loads are B of kt + 2)
            ldsBarrier();
            const uint32_t vA = FULL ? STAGE_KB : validOf(kt + 2u), vB = FULL ? STAGE_KB : validOf(kt + 3u);
            const i32x4    rsrcA = stageRsrc8(A_KCONTIG, refillA, vA, p.lda), rsrcB = stageRsrc8(B_KCONTIG, refillB, vB, p.ldb);
            if(FULL || kt + 3u < numStages)
                refillA += gStageA;
            if(FULL || kt + 4u < numStages)
                refillB += gStageB;
            // Q3: A high x B high (row by row, in the order A arrived); next A low arrives; A refill
#pragma unroll
            for(uint32_t n = 0; n < NQ; ++n)
            {
                mfma16f8<E5M2>(acc[H + n / H][H + n % H], bHi[n % H], aHi[n / H]);
                readSlotA(aLo, aNxt, 0, n);
                loadSlot(full, A_KCONTIG, rsrcA, gOffA, gStepA, kByteA, vA, aCur, n);
                __builtin_amdgcn_sched_barrier(0);
            }
            // Q4: A high x B low; next B low arrives in the registers B high has left; B refill
#pragma unroll
            for(uint32_t n = 0; n < NQ; ++n)
            {
                mfma16f8<E5M2>(acc[H + n % H][n / H], bLo[n / H], aHi[n % H]);
                readSlotB(bHi, bNxt, 0, n);
                loadSlot(full, B_KCONTIG, rsrcB, gOffB, gStepB, kByteB, vB, bCur, n);
                __builtin_amdgcn_sched_barrier(0);
            }
        };

        // prologue: stages 0 and 1 and the B half of stage 2 requested; stage 0 published
        issueHalf(A_KCONTIG, stageAddr(gA, gStageA, 0u), gOffA, gStepA, kByteA, p.lda, validOf(0u), A_AT[0]);
        issueHalf(B_KCONTIG, stageAddr(gB, gStageB, 0u), gOffB, gStepB, kByteB, p.ldb, validOf(0u), B_AT[0]);
        issueHalf(A_KCONTIG, stageAddr(gA, gStageA, 1u), gOffA, gStepA, kByteA, p.lda, validOf(1u), A_AT[1]);
        issueHalf(B_KCONTIG, stageAddr(gB, gStageB, 1u), gOffB, gStepB, kByteB, p.ldb, validOf(1u), B_AT[1]);
        issueHalf(B_KCONTIG, stageAddr(gB, gStageB, 2u), gOffB, gStepB, kByteB, p.ldb, validOf(2u), B_AT[2]);
        refillA = stageAddr(gA, gStageA, 2u), refillB = stageAddr(gB, gStageB, 3u);
        waitVmcnt<3u * WB>();
        ldsBarrier();
        R355_STAMP(1);
#pragma unroll
        for(uint32_t n = 0; n < NQ; ++n)
        {
            readSlotA(aLo, A_AT[0], 0, n);
            readSlotB(bX, B_AT[0], 0, n);
        }

        // six stages per trip bring every buffer and both B register groups back to their roles
        // (main part: the trips whose requests, up to stage kt + 8, all are whole stages inside K)
        // (kept to K-contiguous B: with the transposing reads of an N-contiguous B the second copy of the loop costs more
        // than a hundred spilled registers, and without a K-contiguous operand there is no select to lose)
        const uint32_t wholeStages = B_KCONTIG ? p.k / STAGE_KB : 0u;
        const uint32_t mainTrips   = wholeStages > 8u ? (wholeStages - 8u + 5u) / 6u : 0u;
        using Main = std::true_type;
        using Tail = std::false_type;
        uint32_t kt = 0;
        for(uint32_t trips = mainTrips; trips > 0; --trips, kt += 6u)
        {
            stageBody(Main{}, kt, A_AT[0], A_AT[1], B_AT[0], B_AT[1], bX, bY);
            stageBody(Main{}, kt + 1u, A_AT[1], A_AT[0], B_AT[1], B_AT[2], bY, bX);
            stageBody(Main{}, kt + 2u, A_AT[0], A_AT[1], B_AT[2], B_AT[0], bX, bY);
            stageBody(Main{}, kt + 3u, A_AT[1], A_AT[0], B_AT[0], B_AT[1], bY, bX);
            stageBody(Main{}, kt + 4u, A_AT[0], A_AT[1], B_AT[1], B_AT[2], bX, bY);
            stageBody(Main{}, kt + 5u, A_AT[1], A_AT[0], B_AT[2], B_AT[0], bY, bX);
        }
        for(uint32_t trips = numStages / 6u - mainTrips; trips > 0; --trips, kt += 6u)
        {
            stageBody(Tail{}, kt, A_AT[0], A_AT[1], B_AT[0], B_AT[1], bX, bY);
            stageBody(Tail{}, kt + 1u, A_AT[1], A_AT[0], B_AT[1], B_AT[2], bY, bX);
            stageBody(Tail{}, kt + 2u, A_AT[0], A_AT[1], B_AT[2], B_AT[0], bX, bY);
            stageBody(Tail{}, kt + 3u, A_AT[1], A_AT[0], B_AT[0], B_AT[1], bY, bX);
            stageBody(Tail{}, kt + 4u, A_AT[0], A_AT[1], B_AT[1], B_AT[2], bX, bY);
            stageBody(Tail{}, kt + 5u, A_AT[1], A_AT[0], B_AT[2], B_AT[0], bY, bX);
        }
        const uint32_t rem = numStages - kt;
        if(rem > 0u)
        {
            stageBody(Tail{}, kt, A_AT[0], A_AT[1], B_AT[0], B_AT[1], bX, bY);
            if(rem > 1u)
            {
                stageBody(Tail{}, kt + 1u, A_AT[1], A_AT[0], B_AT[1], B_AT[2], bY, bX);
                if(rem > 2u)
                {
                    stageBody(Tail{}, kt + 2u, A_AT[0], A_AT[1], B_AT[2], B_AT[0], bX, bY);
                    if(rem > 3u)
                    {
                        stageBody(Tail{}, kt + 3u, A_AT[1], A_AT[0], B_AT[0], B_AT[1], bY, bX);
                        if(rem > 4u)
                            stageBody(Tail{}, kt + 4u, A_AT[0], A_AT[1], B_AT[1], B_AT[2], bX, bY);
                    }
                }
            }
        }

        R355_STAMP(2);
        asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); // the last matrix instructions are still in the pipeline
        waitVmcnt<0>();
        ldsBarrier();
        storeTile16<f32x4, float, WB, WB>(acc, p, tm * TILE + wm * WT, tn * TILE + wn * WT, lane, lds + wave * (WB * 4096u));
        R355_STAMP_END();
    }

    template <bool E5M2, bool A_KCONTIG, bool B_KCONTIG>
    __global__ void __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(1, 1))) gemmTiledKernelF8(Params p)
    {
        gemmTiledF8<E5M2, A_KCONTIG, B_KCONTIG, 8>(p);
    }
    template <bool E5M2, bool A_KCONTIG, bool B_KCONTIG>
    __global__ void __launch_bounds__(THREADS) gemmTiledKernelF8Small(Params p)
    {
        gemmTiledF8<E5M2, A_KCONTIG, B_KCONTIG, 4>(p);
    }

    // experiment switch: R355_I8_WIDE=1 in the environment runs the int8 256 x 256 tile on the eight-wave kernel
    inline bool wideI8()
    {
        static const bool on = [] {
            const char* v = getenv("R355_I8_WIDE");
            return v && v[0] == '1';
        }();
        return on;
    }

    template <Elem E, typename OutT>
    int launchLayouts(bool aK, bool bK, uint32_t tile, const Params& p, hipStream_t stream)
    {
        // every XCD gets ceil(count / 8) tile indices (four workgroups each in a quad launch)
        const uint32_t splits = p.splitStages ? ((p.k * ElemTraits<E>::Bytes + STAGE_KB - 1u) / STAGE_KB + p.splitStages - 1u) / p.splitStages : 1u;
        const dim3     grid(((p.tileCount + 7u) / 8u) * 8u * (p.tileQuad ? 4u : 1u), splits), block(THREADS);
        auto launch = [&](auto aKc, auto bKc) {
            constexpr bool AK = decltype(aKc)::value, BK = decltype(bKc)::value;
            if constexpr(E == Elem::I8)
            {
                if(tile == 128u)
                    hipLaunchKernelGGL((gemmTiledKernelI8Small<OutT, AK, BK>), grid, block, 0, stream, p);
                else if(wideI8())
                    hipLaunchKernelGGL((gemmTiledKernelI8Wide<OutT, AK, BK>), grid, dim3(THREADS_WIDE), 0, stream, p);
                else
                    hipLaunchKernelGGL((gemmTiledKernelI8<OutT, AK, BK>), grid, block, 0, stream, p);
            }
            else if constexpr(E == Elem::E4M3 || E == Elem::E5M2)
            {
                if(tile == 128u)
                    hipLaunchKernelGGL((gemmTiledKernelF8Small<E == Elem::E5M2, AK, BK>), grid, block, 0, stream, p);
                else
                    hipLaunchKernelGGL((gemmTiledKernelF8<E == Elem::E5M2, AK, BK>), grid, block, 0, stream, p);
            }
            else if constexpr(E == Elem::F64)
                hipLaunchKernelGGL((gemmTiledKernelF64Small<AK, BK>), grid, block, 0, stream, p); // 128 x 128 only
            else if constexpr(E == Elem::F32)
            {
                if(tile == 128u)
                    hipLaunchKernelGGL((gemmTiledKernelF32Small<AK, BK>), grid, block, 0, stream, p);
                else
                    hipLaunchKernelGGL((gemmTiledKernelF32<AK, BK>), grid, block, 0, stream, p);
            }
            else if(tile == 128u)
                hipLaunchKernelGGL((gemmTiledKernel16Small<E, OutT, AK, BK>), grid, block, 0, stream, p);
            else if(p.deepPipeline)
                hipLaunchKernelGGL((gemmTiledKernel16Deep<E, OutT, AK, BK>), grid, block, 0, stream, p);
            else
                hipLaunchKernelGGL((gemmTiledKernel16<E, OutT, AK, BK>), grid, block, 0, stream, p);
        };
        using T = std::true_type;
        using F = std::false_type;
        if(aK && bK)
            launch(T{}, T{});
        else if(aK)
            launch(T{}, F{});
        else if(bK)
            launch(F{}, T{});
        else
            launch(F{}, F{});
        return r355::checkLaunch("gemm (macro tile)");
    }

#if R355_TILED_HAS(0)
    using r355::computeUnits;

    // Macro tile edge for a problem.
    // Long K: the 128 x 128 tile is a quarter of the work of the 256 x 256 one at about 0.55 of its efficiency with one
    // workgroup per CU, so it pays when the large tiles would leave most CUs idle: 5 rounds128 < 11 rounds256.
    // Short K (up to 8 stages of 128 bytes): the large tile's prologue, epilogue and the gap between workgroups, which
    // nothing overlaps with one workgroup per CU, weigh as much as its K loop, while the two small workgroups of a CU hide
    // each other's.  There the choice follows a timing model - a launch is a number of rounds over the CUs, a round costs a
    // fixed part plus a part per stage; microseconds fitted to launches of 4096^2 ... 8192^2 with k from 256 to 4096:
    //                              per round     per stage
    //   256 x 256, one per CU      9.5 / 13.9      1.30          (16-bit / 8-bit operands: D is 128 / 256 KiB per tile)
    //   128 x 128, two per CU      3.5 /  5.0    0.84 / 0.88     (a round = both workgroups of a CU; half a round = one)
    // (8-bit operands at 8192^2: the small tile up to k = 1024, +4 % there, +29 % at 512, +50 % at 256; 16-bit: at k = 256
    // only, +7 ... +30 %.)  The large tiling's last round runs on small tiles when it would fill at most half of the CUs
    // (mixedRemainder), and the model prices it that way.
    constexpr double SECOND_LAUNCH = 4.0; // microseconds between the two launches of a mixed tiling
    struct TileCosts
    {
        double round256, stage256, round128, stage128;
    };
    TileCosts tileCosts(int32_t inType)
    {
        return r355::dtypeBytes(inType) == 1u ? TileCosts{13.9, 1.30, 5.0, 0.88} : TileCosts{9.5, 1.30, 3.5, 0.84};
    }
    uint32_t macroTile(const r355_gemm_args& g)
    {
        if(g.kernel == R355_KERNEL_TILED || g.kernel == R355_KERNEL_TILED_DEEP)
            return 256u; // (f64 is then refused by the check)
        if(g.kernel == R355_KERNEL_TILED_128 || g.kernel == R355_KERNEL_TILED_128_SPLITK || g.in_type == R355_F64)
            return 128u; // f64 accumulators only fit the small wave tile
        if(g.in_type == R355_F32)
            return 128u; // bound by the matrix-instruction rate either way (146 TFLOP/s at 4096^2 x 2048 with both
                         // tiles), and four times finer rounds: 6144^2 x 2048 runs at 148 TFLOP/s against 111
        const uint64_t cus  = computeUnits();
        const uint64_t t256 = (uint64_t)((g.m + 255u) / 256u) * ((g.n + 255u) / 256u);
        const uint64_t t128 = (uint64_t)((g.m + 127u) / 128u) * ((g.n + 127u) / 128u);
        if(((t128 + cus - 1u) / cus) * 5u < ((t256 + cus - 1u) / cus) * 11u)
            return 128u;
        const uint64_t stages = ((uint64_t)g.k * r355::dtypeBytes(g.in_type) + STAGE_KB - 1u) / STAGE_KB;
        if(stages > 8u)
            return 256u; // (at 16 stages the model still picks the small tile now and then where the large one is 3 - 9 % faster)
        const TileCosts c       = tileCosts(g.in_type);
        const double    tile256 = c.round256 + c.stage256 * static_cast<double>(stages);
        const double    pair128 = c.round128 + c.stage128 * static_cast<double>(stages);
        auto            rounds128 = [&](uint64_t tiles) { return 0.5 * static_cast<double>((tiles + cus - 1u) / cus); };
        const uint64_t  full = t256 / cus, rest = t256 % cus;
        double          cost256 = static_cast<double>(full) * tile256;
        if(rest != 0u)
            cost256 += (g.kernel == R355_KERNEL_AUTO && full > 0u && rest <= cus / 2u) ? rounds128(4u * rest) * pair128 + SECOND_LAUNCH
                                                                                      : tile256;
        return rounds128(t128) * pair128 < cost256 ? 128u : 256u;
    }

    // 16-bit operands on the 256 x 256 tile: the five-buffer K loop when asked for, when A and B (as they lie in memory,
    // leading dimensions included) do not fit the memory-side cache together, or when K is short (its prologue has two
    // stages in flight instead of one: +4 % at k = 512 ... 768, +1 % at 1536, nothing from 2048 on) - gemmTiledKernel16Deep.
    constexpr uint64_t MEMORY_SIDE_CACHE_BYTES = uint64_t{256} << 20;
    bool deepPipeline(const r355_gemm_args& g)
    {
        if(r355::dtypeBytes(g.in_type) != 2u || macroTile(g) != 256u)
            return false;
        if(g.kernel == R355_KERNEL_TILED_DEEP || (uint64_t)g.k * 2u <= 24u * STAGE_KB)
            return true;
        const uint64_t bytesA = (uint64_t)(g.layout_a == R355_ROW_MAJOR ? g.m : g.k) * g.lda * 2u;
        const uint64_t bytesB = (uint64_t)(g.layout_b == R355_ROW_MAJOR ? g.k : g.n) * g.ldb * 2u;
        return bytesA + bytesB > MEMORY_SIDE_CACHE_BYTES;
    }

    // ------------------------------------------------------------------------------------------
    // Split-K.  A problem with few output tiles and a long K (m <= 64 against n, k in the thousands; 512 x 512 x 32768)
    // leaves most CUs idle with one workgroup per tile.  With a caller-provided workspace the 128 x 128 tile kernels run
    // `splits` workgroup rows, each over its own range of K stages, writing partial results in the accumulator type
    // to workspace[split][m][n]; splitKReduceKernel then adds the partial results in split order (deterministic) and applies
    // alpha, beta and C once, exactly as the single-pass epilogue does.
    uint32_t accBytes(int32_t inType)
    {
        return inType == R355_F64 ? 8u : 4u;
    }
    // number of K splits for a problem, 1 = no split; kernel selectors other than AUTO and TILED_128_SPLITK never split.
    // sizing: a query may offer workspace_bytes without a workspace to learn what a launch would use
    uint32_t splitCount(const r355_gemm_args& g, bool sizing = false)
    {
        if(g.kernel != R355_KERNEL_AUTO && g.kernel != R355_KERNEL_TILED_128_SPLITK)
            return 1u;
        if(g.workspace ? !r355::aligned(g.workspace, 16) : !sizing)
            return 1u;
        const uint32_t cus = computeUnits();
        const uint64_t tiles = (uint64_t)((g.m + 127u) / 128u) * ((g.n + 127u) / 128u);
        const uint32_t stages = (g.k * r355::dtypeBytes(g.in_type) + STAGE_KB - 1u) / STAGE_KB;
        if(tiles * 2u > cus || stages < 16u)
            return 1u;
        // one workgroup per CU (two per CU, which the 80 KiB of LDS allow, measured 5 - 20 % slower), at least 8 stages per share
        uint32_t splits = static_cast<uint32_t>(cus / tiles);
        splits = splits < stages / 8u ? splits : stages / 8u;
        splits = splits < 32u ? splits : 32u;
        if(splits < 2u)
            return 1u;
        // shares are whole stages; recompute the count from the share so that no share is empty
        const uint32_t share = (stages + splits - 1u) / splits;
        splits               = (stages + share - 1u) / share;
        if(splits < 2u || (uint64_t)splits * g.m * g.n * accBytes(g.in_type) > g.workspace_bytes)
            return 1u;
        return splits;
    }
    uint32_t splitStagesOf(const r355_gemm_args& g, uint32_t splits)
    {
        const uint32_t stages = (g.k * r355::dtypeBytes(g.in_type) + STAGE_KB - 1u) / STAGE_KB;
        return (stages + splits - 1u) / splits;
    }

    // One thread per 4 consecutive columns of a row of D (n is a multiple of 16).  AccT: f32, i32 or f64.
    template <typename AccT, typename OutT>
    __global__ void __launch_bounds__(256) splitKReduceKernel(const AccT* __restrict__ ws, uint32_t splits, uint64_t sliceElems, uint32_t m,
                                                              uint32_t n, const OutT* c, uint32_t ldc, OutT* d, uint32_t ldd, double alphaD,
                                                              double betaD)
    {
        const uint64_t idx = (uint64_t)blockIdx.x * 256u + threadIdx.x; // 4-column group
        const uint32_t groupsPerRow = n / 4u;
        if(idx >= (uint64_t)m * groupsPerRow)
            return;
        const uint32_t row = static_cast<uint32_t>(idx / groupsPerRow), col = static_cast<uint32_t>(idx % groupsPerRow) * 4u;
        using AccV = AccT __attribute__((ext_vector_type(4)));
        using OutV = OutT __attribute__((ext_vector_type(4)));
        const AccT* mine = ws + (uint64_t)row * n + col;
        AccV        sum  = *reinterpret_cast<const AccV*>(mine);
        // up to eight partial results requested at a time, added in split order (the order never depends on timing)
        for(uint32_t s = 1; s < splits; s += 8u)
        {
            const uint32_t count = splits - s < 8u ? splits - s : 8u; // uniform
            AccV           v[8];
#pragma unroll
            for(uint32_t u = 0; u < 8; ++u)
                if(u < count)
                    v[u] = *reinterpret_cast<const AccV*>(mine + (s + u) * sliceElems);
#pragma unroll
            for(uint32_t u = 0; u < 8; ++u)
                if(u < count)
                {
#pragma unroll
                    for(uint32_t e = 0; e < 4; ++e)
                        sum[e] += v[u][e];
                }
        }
        const AccT alpha = static_cast<AccT>(alphaD), beta = static_cast<AccT>(betaD);
        OutV       out;
        if(beta != static_cast<AccT>(0))
        {
            const OutV cv = *reinterpret_cast<const OutV*>(c + (uint64_t)row * ldc + col);
#pragma unroll
            for(uint32_t e = 0; e < 4; ++e)
                out[e] = static_cast<OutT>(alpha * sum[e] + beta * static_cast<AccT>(cv[e]));
        }
        else
        {
#pragma unroll
            for(uint32_t e = 0; e < 4; ++e)
                out[e] = static_cast<OutT>(alpha * sum[e]);
        }
        *reinterpret_cast<OutV*>(d + (uint64_t)row * ldd + col) = out;
    }

    // Mixed tiling (R355_KERNEL_AUTO only).  A problem of a few rounds whose last round of 256 x 256 tiles would
    // occupy at most half of the CUs runs that last part on 128 x 128 tiles instead, in a second launch: four small
    // tiles per large one, two workgroups per CU, together about 0.4 (up to a quarter of the CUs' worth of large
    // tiles) or 0.6 of a large-tile round instead of a whole one.  Returns the number of 256 x 256 tile indices the
    // second launch covers, 0 for a single launch.
    uint32_t mixedRemainder(const r355_gemm_args& g)
    {
        if(g.kernel != R355_KERNEL_AUTO || g.in_type == R355_F32 || g.in_type == R355_F64 || macroTile(g) != 256u)
            return 0u;
        const uint32_t cus   = computeUnits();
        const uint32_t total = ((g.m + 255u) / 256u) * ((g.n + 255u) / 256u);
        const uint32_t rest  = total % cus;
        return (total > cus && rest != 0u && rest <= cus / 2u) ? rest : 0u;
    }
#endif // part 0
} // namespace

namespace r355
{
#if R355_TILED_HAS(0)
    int splitKReduce(const r355_gemm_args& g, const GemmTileParams& p, uint32_t splits, hipStream_t stream)
    {
        // p is the kernel's view of the problem (D row-major m x n; a col-major D runs as its transpose)
        const uint64_t groups = (uint64_t)p.m * (p.n / 4u);
        const dim3     grid(static_cast<uint32_t>((groups + 255u) / 256u)), block(256);
        const uint64_t slice = (uint64_t)p.m * p.n;
        auto go = [&](auto acc, auto out) {
            using AccT = decltype(acc);
            using OutT = decltype(out);
            hipLaunchKernelGGL((splitKReduceKernel<AccT, OutT>), grid, block, 0, stream, static_cast<const AccT*>(g.workspace), splits, slice,
                               p.m, p.n, reinterpret_cast<const OutT*>(p.c), p.ldc, reinterpret_cast<OutT*>(p.d), p.ldd, p.alpha, p.beta);
        };
        switch(g.out_type)
        {
        case R355_F16: go(0.0f, _Float16{}); break;
        case R355_BF16: go(0.0f, __bf16{}); break;
        case R355_F32: go(0.0f, 0.0f); break;
        case R355_F64: go(0.0, 0.0); break;
        case R355_I32: go(int{}, int{}); break;
        default: go(int{}, static_cast<signed char>(0)); break; // int8 result: the low byte, as the single-pass epilogue narrows it
        }
        return checkLaunch("gemm (split-K reduction)");
    }

    int gemmTiledCheck(const r355_gemm_args& g, r355_gemm_plan* plan)
    {
        const bool pairOk = (g.in_type == R355_F16 && (g.out_type == R355_F16 || g.out_type == R355_F32))
                            || (g.in_type == R355_BF16 && (g.out_type == R355_BF16 || g.out_type == R355_F32))
                            || ((g.in_type == R355_E4M3 || g.in_type == R355_E5M2) && g.out_type == R355_F32)
                            || (g.in_type == R355_F32 && g.out_type == R355_F32)
                            || (g.in_type == R355_F64 && g.out_type == R355_F64)
                            || (g.in_type == R355_I8 && (g.out_type == R355_I32 || g.out_type == R355_I8));
        if(!pairOk)
            return fail(R355_ERR_UNSUPPORTED, "tiled gemm: no kernel for in_type %d -> out_type %d", g.in_type, g.out_type);
        const uint32_t es = dtypeBytes(g.in_type), os = dtypeBytes(g.out_type);
        const uint32_t tile = macroTile(g);
        if(g.in_type == R355_F64 && tile != 128u)
            return fail(R355_ERR_UNSUPPORTED, "tiled gemm: f64 runs the 128 x 128 macro tile only");
        if(g.beta != 0.0 && g.layout_c != g.layout_d)
            return fail(R355_ERR_UNSUPPORTED, "tiled gemm: C and D must share an orientation");
        const uint32_t tk = STAGE_KB / es;
        // K moves in 16-byte chunks; a last K stage that is not full is completed with zeros by the loads
        const bool     fiveBuffers = es != 2 || deepPipeline(g);
        const uint32_t kGranule    = CHUNK / es;
        if(g.m % 16 || g.n % 16 || g.m == 0 || g.n == 0 || g.k % kGranule || g.k == 0)
            return fail(R355_ERR_BAD_SIZE, "tiled gemm: m=%u n=%u must be multiples of 16 and k=%u of %u", g.m, g.n, g.k, kGranule);
        // lane offsets are 32-bit (255 rows of ld elements; the epilogue's: 128 rows of C / D) and a K stage of an
        // M/N-contiguous operand is one buffer
        if((uint64_t)g.lda * es > (1u << 23) || (uint64_t)g.ldb * es > (1u << 23) || (uint64_t)g.ldd * os > (1u << 23)
           || (g.beta != 0.0 && (uint64_t)g.ldc * os > (1u << 23)))
            return fail(R355_ERR_UNSUPPORTED, "tiled gemm: leading dimensions above 8 MiB per row / column");
        if(!aligned(g.a, 16) || !aligned(g.b, 16) || (g.lda * es) % 16 || (g.ldb * es) % 16 || !aligned(g.d, 16)
           || (g.ldd * os) % 16 || (g.beta != 0.0 && (!aligned(g.c, 16) || (g.ldc * os) % 16)))
            return fail(R355_ERR_MISALIGNED, "tiled gemm: pointers and leading dimensions of A, B, C, D must keep 16-byte alignment");
        if(plan)
        {
            plan->kernel       = R355_KERNEL_TILED;
            plan->macro_tile_m = tile;
            plan->macro_tile_n = tile;
            plan->macro_tile_k = tk;
            // with mixed tiling: the first launch (the second covers mixedRemainder(g) tile indices on 128 x 128 tiles)
            plan->grid_x       = ((((g.m + tile - 1) / tile) * ((g.n + tile - 1) / tile) - mixedRemainder(g) + 7u) / 8u) * 8u;
            plan->grid_y       = 1;
            plan->block_x      = THREADS;
            plan->block_y      = 1;
            plan->lds_bytes    = (fiveBuffers || tile == 128u ? 5u * OPER_BYTES : NUM_STAGES * STAGE_BYTES) * tile / 256u;
            const uint32_t splits = tile == 128u ? splitCount(g, true) : 1u;
            plan->split_k         = splits;
            plan->grid_y          = splits;
            plan->workspace_bytes = splits > 1u ? (uint64_t)splits * g.m * g.n * accBytes(g.in_type) : 0u;
        }
        if(g.kernel == R355_KERNEL_TILED_128_SPLITK && splitCount(g, plan != nullptr) < 2u)
            return fail(R355_ERR_BAD_SIZE,
                        "tiled gemm (split-K): needs a workspace of splits x m x n accumulator elements (r355_gemm_query with a large "
                        "workspace_bytes reports the size), at most half as many 128 x 128 tiles as CUs and k of at least 16 stages of 128 bytes");
        return R355_OK;
    }

    int gemmTiledLaunch(const r355_gemm_args& g, hipStream_t stream)
    {
        // The kernel writes D row-major.  A col-major D (and C) is the row-major transpose:
        // D^T = B^T A^T, i.e. swap the operands and the roles of m and n; an operand's
        // K-contiguity is unchanged by the swap.
        const bool dRow = g.layout_d == R355_ROW_MAJOR;
        Params     p;
        p.k = g.k;
        p.c = static_cast<const char*>(g.c), p.d = static_cast<char*>(g.d);
        p.ldc = g.ldc, p.ldd = g.ldd;
        p.alpha = g.alpha, p.beta = g.beta;
        bool aK, bK;
        if(dRow)
        {
            p.m = g.m, p.n = g.n;
            p.a = static_cast<const char*>(g.a), p.b = static_cast<const char*>(g.b);
            p.lda = g.lda, p.ldb = g.ldb;
            aK = g.layout_a == R355_ROW_MAJOR, bK = g.layout_b == R355_COL_MAJOR;
        }
        else
        {
            p.m = g.n, p.n = g.m;
            p.a = static_cast<const char*>(g.b), p.b = static_cast<const char*>(g.a);
            p.lda = g.ldb, p.ldb = g.lda;
            aK = g.layout_b == R355_COL_MAJOR, bK = g.layout_a == R355_ROW_MAJOR;
        }
        const uint32_t tile = macroTile(g);
        p.tilesM = (p.m + tile - 1) / tile, p.tilesN = (p.n + tile - 1) / tile;
        p.tileFirst = 0u, p.tileCount = p.tilesM * p.tilesN, p.tileQuad = 0u;
        auto part = [&](uint32_t t, const Params& q) {
            switch(g.in_type)
            {
            case R355_F16: return gemmTiledPart0(g, aK, bK, t, q, stream);
            case R355_BF16: return gemmTiledPart1(g, aK, bK, t, q, stream);
            case R355_E4M3:
            case R355_E5M2:
            case R355_I8: return gemmTiledPart2(g, aK, bK, t, q, stream);
            case R355_F32:
            case R355_F64: return gemmTiledPart3(g, aK, bK, t, q, stream);
            default: return fail(R355_ERR_UNSUPPORTED, "tiled gemm: unknown in_type %d", g.in_type);
            }
        };
        p.splitStages = 0u, p.splitStrideD = 0u;
        p.deepPipeline = deepPipeline(g) ? 1u : 0u;
        static const uint32_t staggerTicks = [] {
            const char* v = getenv("R355_STAGGER_TICKS");
            return v ? static_cast<uint32_t>(atoi(v)) : 0u;
        }();
        p.stagger = staggerTicks, p.staggerBlocks = computeUnits();
        const uint32_t splits = tile == 128u ? splitCount(g) : 1u;
        if(splits > 1u)
        {
            // partial results in the accumulator type, row-major with leading dimension n, alpha = 1 and beta = 0; the
            // reduction applies the caller's scalars and C
            Params q        = p;
            q.splitStages   = splitStagesOf(g, splits);
            q.splitStrideD  = (uint64_t)p.m * p.n * accBytes(g.in_type);
            q.d             = static_cast<char*>(g.workspace);
            q.ldd           = p.n;
            q.c             = nullptr;
            q.alpha = 1.0, q.beta = 0.0;
            r355_gemm_args ga = g; // the kernels of the accumulator-typed output
            ga.out_type       = g.in_type == R355_F64 ? R355_F64 : (g.in_type == R355_I8 ? R355_I32 : R355_F32);
            const int rc      = [&] {
                switch(g.in_type)
                {
                case R355_F16: return gemmTiledPart0(ga, aK, bK, 128u, q, stream);
                case R355_BF16: return gemmTiledPart1(ga, aK, bK, 128u, q, stream);
                case R355_E4M3:
                case R355_E5M2:
                case R355_I8: return gemmTiledPart2(ga, aK, bK, 128u, q, stream);
                default: return gemmTiledPart3(ga, aK, bK, 128u, q, stream);
                }
            }();
            return rc != R355_OK ? rc : splitKReduce(g, p, splits, stream);
        }
        const uint32_t rest = mixedRemainder(g);
        if(rest == 0u)
            return part(tile, p);
        // whole rounds on 256 x 256 tiles, then the rest of the walk on 128 x 128 tiles, four per index
        Params big = p, small = p;
        big.tileCount   = p.tileCount - rest;
        small.tileFirst = big.tileCount, small.tileCount = rest, small.tileQuad = 1u;
        const int rc = part(256u, big);
        return rc != R355_OK ? rc : part(128u, small);
    }
#endif // part 0

#if R355_TILED_HAS(0)
    int gemmTiledPart0(const r355_gemm_args& g, bool aK, bool bK, uint32_t tile, const GemmTileParams& p, hipStream_t stream)
    {
        return g.out_type == R355_F16 ? launchLayouts<Elem::F16, _Float16>(aK, bK, tile, p, stream)
                                      : launchLayouts<Elem::F16, float>(aK, bK, tile, p, stream);
    }
#endif
#if R355_TILED_HAS(1)
    int gemmTiledPart1(const r355_gemm_args& g, bool aK, bool bK, uint32_t tile, const GemmTileParams& p, hipStream_t stream)
    {
        return g.out_type == R355_BF16 ? launchLayouts<Elem::BF16, __bf16>(aK, bK, tile, p, stream)
                                       : launchLayouts<Elem::BF16, float>(aK, bK, tile, p, stream);
    }
#endif
#if R355_TILED_HAS(2)
    int gemmTiledPart2(const r355_gemm_args& g, bool aK, bool bK, uint32_t tile, const GemmTileParams& p, hipStream_t stream)
    {
        if(g.in_type == R355_E4M3)
            return launchLayouts<Elem::E4M3, float>(aK, bK, tile, p, stream);
        if(g.in_type == R355_E5M2)
            return launchLayouts<Elem::E5M2, float>(aK, bK, tile, p, stream);
        return g.out_type == R355_I32 ? launchLayouts<Elem::I8, int>(aK, bK, tile, p, stream)
                                      : launchLayouts<Elem::I8, signed char>(aK, bK, tile, p, stream);
    }
#endif
#if R355_TILED_HAS(3)
    int gemmTiledPart3(const r355_gemm_args& g, bool aK, bool bK, uint32_t tile, const GemmTileParams& p, hipStream_t stream)
    {
        return g.in_type == R355_F32 ? launchLayouts<Elem::F32, float>(aK, bK, tile, p, stream)
                                     : launchLayouts<Elem::F64, double>(aK, bK, tile, p, stream);
    }
#endif
} // namespace r355
