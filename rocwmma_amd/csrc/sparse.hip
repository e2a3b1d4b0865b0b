// 2:4 structured-sparse GEMM on gfx950 sparse matrix cores (v_smfmac_*), plus the host-side
// compressor.  The reference has no sparse path; the storage format is defined here (and, for device code,
// in rocwmma/rocwmma_sparse.hpp, which also documents the operand formats of the instructions).
//
// A (m x k, 1-byte elements, or f16 / bf16 for the block-per-wave kernel) keeps 2 of every aligned group of 4
// along k and is stored K-blocked: a stage is 128 dense bytes of k, and with ES the element size
//   values  [stage][row / 16][lane group g = 0..3][row % 16][16 bytes]   kept elements of dense
//           k in [stage * 128 / ES + g * 32 / ES, ... + 32 / ES) of the row, in position order
//   meta    the same indexing with 4 / ES bytes: one nibble idx0 | idx1 << 2 (idx0 < idx1) per group of 4,
//           the lane's first group in the lowest bits = the index register of v_smfmac_*_16x16x(128 / ES)
// so that all a 256-row macro tile needs of one stage is 16 + 4 KiB of consecutive bytes (whole cache lines;
// with row-major compressed rows a stage touched 64 + 16 bytes of every row's lines and the direct-to-LDS
// loads ran at two thirds of the rate), and a fragment's 16 bytes per lane are consecutive across lanes.
// B is dense, in either orientation (the macro tile stages a col-major B as rows and a row-major B as k-rows); D row- or
// col-major.  m % 16 == 0, k % (128 / ES) == 0.
//
// Two kernels:
//   sparseTiledKernel    256 x 256 macro tile, one K step of 128 bytes per stage, a ring of three LDS slots filled
//                        by direct-to-LDS loads two stages ahead (kept values 16 KiB + indices 4 or 2 KiB
//                        + dense B 32 KiB per stage), 2 x 2 waves with 8 x 8 accumulators of
//                        v_smfmac_*_16x16x128 (int8, e4m3) or v_smfmac_f32_16x16x64 (f16, bf16) each (under the
//                        board's power limit the register-resident int8 loop of this shape sustains 7.5 POP/s
//                        against 6.5 for 32x32x64); a stage is split into quadrants of the wave tile as in the
//                        dense fp8 kernel; the result is transposed through LDS so that D leaves in whole
//                        rows.  Edge tiles (m, n multiples of 16): rows of A and B beyond the matrix lie outside
//                        the stage's buffers and load as zeros, the epilogue stores what is inside D.
//   sparseBlockPerWave   one 16 x 16 or 32 x 32 block of D per wave through the sparse fragment API
//                        (rocwmma_sparse.hpp) straight from global memory; fallback for shapes that do not fill a
//                        macro tile.
//
// Measurement builds of the macro-tile kernel (`python -m rocwmma_amd.build --variant <name> -D<macro> ...` puts a
// second library under lib/variant_<name>/; never the shipped one - the first three compute wrong results on purpose):
//   R355_ABLATE_MFMA    no matrix instructions (data movement alone)
//   R355_ABLATE_READS   no LDS reads of the operands
//   R355_ABLATE_LOADS   no direct loads after the prologue's
//   R355_SPARSE_A_DIRECT  every wave takes the kept values and indices of its own 128 rows straight from global memory
//                       into registers, one stage ahead, and only B goes through LDS (results correct).  Measured
//                       12 - 26 % slower: the two waves that share a block row both fetch it, so 72 instead of 52 KiB
//                       per stage pass the CU's vector-memory path, which is what bounds this kernel.
#include <hip/hip_runtime.h>

#include <cstring>

#include <rocwmma/rocwmma_sparse.hpp>

#include "common.hpp"
#include "lds_dma.hpp"
#include "operand_tile.hpp"
#include "tile_map.hpp"

namespace
{
    using namespace rocwmma;
    using i32x4 = int __attribute__((ext_vector_type(4)));
    using i32x8 = int __attribute__((ext_vector_type(8)));
    using f32x4 = float __attribute__((ext_vector_type(4)));

    constexpr uint32_t WAVES_X = 2, WAVES_Y = 2;

    // ------------------------------------------------------------------ block per wave, on the fragment API
    template <typename InT, typename AccE, uint32_t Blk>
    __global__ void __launch_bounds__(WAVES_X* WAVES_Y * 64) sparseBlockPerWave(uint32_t       m,
                                                                               uint32_t       n,
                                                                               uint32_t       k,
                                                                               const InT*     aVals,
                                                                               const uint8_t* aMeta,
                                                                               const InT*     b,
                                                                               const AccE*    c,
                                                                               AccE*          d,
                                                                               uint32_t       ldb,
                                                                               uint32_t       ldc,
                                                                               uint32_t       ldd,
                                                                               layout_t       layoutB,
                                                                               layout_t       layoutC,
                                                                               layout_t       layoutD,
                                                                               AccE           alpha,
                                                                               AccE           beta)
    {
        using S                 = Sparse24<InT>;
        constexpr uint32_t BK   = S::StageK; // one stage per trip
        using FragA             = fragment<sparse_matrix_a, Blk, Blk, BK, InT, row_major>;
        using FragMeta          = fragment<sparse_metadata, Blk, Blk, BK, InT>;
        using FragB             = fragment<matrix_b, Blk, Blk, BK, InT>; // orientation given at run time
        using FragAcc           = fragment<accumulator, Blk, Blk, BK, AccE>;
        const uint32_t row = (blockIdx.x * WAVES_X + threadIdx.x / 64u) * Blk;
        const uint32_t col = (blockIdx.y * WAVES_Y + threadIdx.y) * Blk;
        if(row >= m || col >= n)
            return;
        const InT*     pa = aVals + S::valueOffset(row, 0u, m);
        const uint8_t* pm = aMeta + S::metaOffset(row, 0u, m);
        const bool     bCol = layoutB == mem_col_major;
        const InT*     pb   = bCol ? b + (uint64_t)col * ldb : b + col;
        const uint64_t stepB = bCol ? (uint64_t)BK : (uint64_t)BK * ldb; // one stage further along k
        const uint32_t strideV = S::valueStageStride(m), strideM = S::metaStageStride(m);

        FragA    fragA;
        FragMeta fragMeta;
        FragB    fragB;
        FragAcc  fragAcc;
        fill_fragment(fragAcc, static_cast<AccE>(0));
        for(uint32_t kk = 0; kk < k; kk += BK)
        {
            load_matrix_sync(fragA, pa, strideV);
            load_matrix_sync(fragMeta, pm, strideM);
            load_matrix_sync(fragB, pb, ldb, layoutB);
            mma_sync(fragAcc, fragA, fragMeta, fragB, fragAcc);
            pa += strideV, pm += strideM, pb += stepB;
        }
        const uint64_t offC = layoutC == mem_row_major ? (uint64_t)row * ldc + col : (uint64_t)col * ldc + row;
        const uint64_t offD = layoutD == mem_row_major ? (uint64_t)row * ldd + col : (uint64_t)col * ldd + row;
        if(beta != static_cast<AccE>(0))
        {
            FragAcc fragC;
            load_matrix_sync(fragC, c + offC, ldc, layoutC);
#pragma unroll
            for(uint32_t i = 0; i < FragAcc::num_elements; ++i)
                fragAcc.x[i] = alpha * fragAcc.x[i] + beta * fragC.x[i];
        }
        else
        {
#pragma unroll
            for(uint32_t i = 0; i < FragAcc::num_elements; ++i)
                fragAcc.x[i] = alpha * fragAcc.x[i];
        }
        store_matrix_sync(d + offD, fragAcc, ldd, layoutD);
    }

    // ------------------------------------------------------------------ macro-tile kernels
    // WB = accumulator blocks per wave-tile edge: 8 - macro tile 256 x 256, one workgroup per CU; 4 - macro tile 128 x 128,
    // two workgroups per CU, for problems whose large tiles would leave most CUs idle.
    constexpr uint32_t T_K = 128; // dense bytes of K per stage
    constexpr uint32_t T_THREADS = 256;
    template <uint32_t WB>
    struct SpTile
    {
        static constexpr uint32_t M = 32u * WB, N = 32u * WB;
        static constexpr uint32_t A_BYTES     = M * (T_K / 2); // kept values: 16 / 8 KiB
        static constexpr uint32_t META_BYTES  = M * (T_K / 8); // indices: 4 / 2 KiB (half of them used by 2-byte elements)
        static constexpr uint32_t B_BYTES     = N * T_K; // dense B: 32 / 16 KiB
        static constexpr uint32_t OFF_META    = A_BYTES;
        static constexpr uint32_t OFF_B       = A_BYTES + META_BYTES;
        static constexpr uint32_t STAGE_BYTES = A_BYTES + META_BYTES + B_BYTES; // 52 / 26 KiB
        // direct loads of 4 KiB (256 lanes x 16 bytes) per stage: NA of kept values, one of indices - issued by the first
        // META_WAVES waves only, 1 KiB each, so that nothing lands beyond the index region - and NB of B
        static constexpr uint32_t NA = A_BYTES / 4096u, NB = B_BYTES / 4096u, LOADS = NA + 1u + NB; // 13 / 7
        static constexpr uint32_t META_WAVES = META_BYTES / 1024u; // 4 / 2
        // how a stage's loads are dealt out over the four quadrants after the barrier that frees their slot (Q3, Q4 of that
        // stage, Q1, Q2 of the next): load i of a quadrant goes out in its slot i * STEP + 1
        //   large tile: 4 + 3 | 3 + 3 loads, every 4th / 5th slot of a quadrant's 16; small tile: 2 + 2 | 2 + 1, every 2nd of 4
        static constexpr uint32_t FIRST_HALF = WB == 8 ? 7u : 4u;
    };

    struct TiledParams
    {
        uint32_t       m, n, k;
        const uint8_t* aVals;
        const uint8_t* aMeta;
        const uint8_t* b;
        const char*    c;
        char*          d;
        uint32_t       ldb, ldc, ldd;
        double         alpha, beta;
        uint32_t       tilesM, tilesN;
        uint32_t       dRow; // D (and C) row-major
    };

    // Three stage slots (3 x 52 = 156 of 160 KiB; small tile: 3 x 26 = 78 KiB): the slot of stage kt is refilled with stage
    // kt + 3 once every wave has its operands in registers, so one and a half to two stages of loads are in flight at
    // any time.  The direct loads are explicit (lds_dma.hpp) and the only vmcnt wait is "all but the youngest stage's
    // loads" before each barrier; loads past the last stage are issued with nothing in range (zero fill, no memory
    // traffic), so every stage issues the same loads.
    //
    // A stage is one 128-byte K step: WB x WB matrix instructions per wave.  As in the dense fp8 kernel it is split
    // into quadrants of the wave tile, consecutive quadrants sharing one operand group of H = WB / 2 blocks:
    //     Q1 = A[lo] x B[lo]   Q2 = A[lo] x B[hi]   Q3 = A[hi] x B[hi]   Q4 = A[hi] x B[lo]
    //     under Q1: B[hi] of this stage arrives      under Q3: A[lo] of the next stage
    //     under Q2: A[hi] of this stage              under Q4: B[lo] of the next stage
    // After Q2 the stage's slot is no longer read: barrier, then its refill - the first half of stage kt + 3's loads under
    // Q3 and Q4, the rest under Q1 and Q2 of the next stage, so that the memory pipeline has requests to work on during the
    // whole stage (all of them under Q3 and Q4: 0.0722 ms for 4096 x 4096 x 8192 int8 against 0.0710).  The two B register
    // groups swap roles every stage and the ring has three slots: six stages per loop trip, single exit, then up to five
    // stages of straight-line code.
    constexpr uint32_t RING = 3;

    template <uint32_t H>
    struct AGroup
    {
        i32x4 v[H]; // 16 kept bytes per lane and block
        int   idx[H];
    };

    enum class SpElem
    {
        I8,
        E4M3,
        F16,
        BF16
    };

    template <SpElem E, typename AccV>
    __device__ __forceinline__ void smfmac16(AccV& acc, const i32x4& a, const i32x8& b, int idx)
    {
        // the accumulator is the instruction's destination and addend at once: updated in place, in an AGPR
        // (2-byte elements: the index bits are the low half of the register, which is what ABID 0 names)
#ifdef R355_ABLATE_MFMA
        asm volatile("" : "+a"(acc) : "v"(a), "v"(b), "v"(idx));
        return;
#endif
        if constexpr(E == SpElem::E4M3)
            asm volatile("v_smfmac_f32_16x16x128_fp8_fp8 %0, %1, %2, %3" : "+a"(acc) : "v"(a), "v"(b), "v"(idx));
        else if constexpr(E == SpElem::I8)
            asm volatile("v_smfmac_i32_16x16x128_i8 %0, %1, %2, %3" : "+a"(acc) : "v"(a), "v"(b), "v"(idx));
        else if constexpr(E == SpElem::F16)
            asm volatile("v_smfmac_f32_16x16x64_f16 %0, %1, %2, %3" : "+a"(acc) : "v"(a), "v"(b), "v"(idx));
        else
            asm volatile("v_smfmac_f32_16x16x64_bf16 %0, %1, %2, %3" : "+a"(acc) : "v"(a), "v"(b), "v"(idx));
    }

    // B_KCONTIG: B is col-major (K contiguous: rows of the tile in LDS, one ds_read_b128 per 16-byte piece); otherwise
    // row-major (N contiguous: k-rows in LDS, swizzled and read back with transposing reads as the dense kernels' M/N-
    // contiguous operands are, operand_tile.hpp: two reads per piece).
    template <SpElem E, bool B_KCONTIG, uint32_t WB>
    __device__ __forceinline__ void sparseTiled(const TiledParams& p)
    {
        using T = SpTile<WB>;
        constexpr bool     INT = E == SpElem::I8;
        constexpr uint32_t ES  = (E == SpElem::F16 || E == SpElem::BF16) ? 2u : 1u; // element bytes
        constexpr uint32_t H = WB / 2u, NQ = H * H; // blocks per operand group, matrix instructions per quadrant
        constexpr uint32_t OFF_META = T::OFF_META, OFF_B = T::OFF_B, STAGE_BYTES = T::STAGE_BYTES;
        using AccE = std::conditional_t<INT, int, float>;
        using AccV = std::conditional_t<INT, i32x4, f32x4>;
        using AG   = AGroup<H>;
        using r355::loadToLds;
#ifdef R355_SPARSE_A_DIRECT
        static_assert(WB == 8, "the measurement build that keeps A out of LDS has the large tile only");
#endif

        __shared__ __attribute__((aligned(1024))) char lds[RING * STAGE_BYTES];

        uint32_t tm, tn;
        if(!r355::tileCoord(blockIdx.x, p.tilesM, p.tilesN, tm, tn))
            return;

        const uint32_t tid  = threadIdx.x;
        const uint32_t lane = tid & 63u;
        const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const uint32_t wm = wave >> 1, wn = wave & 1u;
        const uint32_t t = lane & 15u, g = lane >> 4;
        const uint32_t ldsBase
            = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) char*)lds));

        // ---- global -> LDS (per thread, fixed).  LDS chunk L = j * 256 + tid of each operand tile.
        //   kept values / indices: the tile's share of a stage is consecutive bytes, copied as they are
        //   dense B: 8 chunks per row, chunk c of row r in slot c ^ ((r >> 1) & 7)
        //   Edge tiles: the tile's rows of A are the first validM / 16 KiB (values) of its share of a stage and the rows
        //   of B the first validN * ldb bytes from the tile's first row: each load's buffer ends exactly there, and what
        //   lies beyond loads as zeros (the raw-buffer range check covers lane offset + scalar offset).
        const uint32_t gOffA = tid * 16u;
        const uint32_t rowB = tid >> 3, slotB = tid & 7u;
        const uint32_t ldbBytes = p.ldb * ES;
        const uint32_t gOffB = rowB * ldbBytes + ((slotB ^ ((rowB >> 1) & 7u)) * 16u), gStepB = 32u * ldbBytes; // (col-major B)
        const uint32_t numStages = p.k * ES / T_K;
        const uint64_t strideV = (uint64_t)p.m * 64u, strideM = (uint64_t)p.m * (16u / ES); // bytes between stages
        // (wave-uniform; the readfirstlane calls only tell the compiler so, which keeps the buffer descriptors in scalar registers)
        const uint32_t validM = __builtin_amdgcn_readfirstlane(p.m - tm * T::M < T::M ? p.m - tm * T::M : T::M);
        const uint32_t validN = __builtin_amdgcn_readfirstlane(p.n - tn * T::N < T::N ? p.n - tn * T::N : T::N);
        const uint64_t gA = r355::uniformAddress(p.aVals + (uint64_t)tm * T::A_BYTES);
        const uint64_t gM = r355::uniformAddress(p.aMeta + (uint64_t)tm * (T::META_BYTES / ES));
        const uint64_t gB = r355::uniformAddress(p.b + (B_KCONTIG ? (uint64_t)tn * T::N * ldbBytes : (uint64_t)tn * T::N * ES));
        const uint32_t dmaDst = ldsBase + wave * 1024u; // lane l lands at dmaDst + slot + piece + 16 l
        // row-major B: a stage is 128 / ES k-rows of the tile's columns; a lane whose 16-byte chunk lies beyond n takes
        // the tile's first chunk instead (what it brings only feeds columns of D that are never stored)
        uint32_t gOffBn[WB] = {}, gStepBn = 0u, kByteBn = 0u;
        uint64_t gStageBn = 0u;
        if constexpr(!B_KCONTIG)
            r355::tile::laneOffsets8<false, WB, ES>(tid, p.ldb, validN, gOffBn, gStepBn, gStageBn, kByteBn);
        const bool metaWave = wave < T::META_WAVES; // (wave-uniform) this wave brings 1 KiB of the stage's indices

        // a buffer of `bytes` bytes at addr, or over nothing for a stage past the end
        auto rsrcOf = [](uint64_t addr, uint32_t bytes, bool valid) {
            return i32x4{static_cast<int>(static_cast<uint32_t>(addr)), static_cast<int>(static_cast<uint32_t>(addr >> 32) & 0xFFFFu),
                         static_cast<int>(valid ? bytes : 0u), 0x00020000};
        };
        // load x of stage `stage` into the slot at byte `at`: NA of kept values, then the indices, then NB of dense B
        auto issueLoad = [&](uint32_t stage, uint32_t at, uint32_t x) {
#ifdef R355_ABLATE_LOADS
            if(stage >= RING)
                return;
#endif
#ifdef R355_SPARSE_A_DIRECT
            if(x <= T::NA)
                return; // A does not pass through LDS
#endif
            const bool     valid = stage < numStages;
            const uint32_t st    = valid ? stage : 0u;
            if(x < T::NA)
                loadToLds(rsrcOf(gA + st * strideV, validM * 64u, valid), gOffA, x * 4096u, dmaDst + at + x * 4096u);
            else if(x == T::NA)
            {
                if(T::META_WAVES == 4u || metaWave)
                    loadToLds(rsrcOf(gM + st * strideM, validM * (16u / ES), valid), gOffA, 0u, dmaDst + at + OFF_META);
            }
            else if constexpr(B_KCONTIG) // 32 rows of B per load; the buffer ends with the tile's last valid row
                loadToLds(rsrcOf(gB + (uint64_t)st * T_K, validN * ldbBytes - st * T_K, valid), gOffB, (x - T::NA - 1u) * gStepB,
                          dmaDst + at + OFF_B + (x - T::NA - 1u) * 4096u);
            else // 16 / ES k-rows of B per load; the buffer is the stage's k-rows (K is whole stages: no tail)
                loadToLds(rsrcOf(gB + st * gStageBn, (T_K / ES) * ldbBytes, valid), gOffBn[x - T::NA - 1u], (x - T::NA - 1u) * gStepBn,
                          dmaDst + at + OFF_B + (x - T::NA - 1u) * 4096u);
        };
        // wait until only the youngest COUNT loads of this wave are outstanding, METAS of which are index loads (which
        // only the first META_WAVES waves issue)
        auto waitYoungest = [&](auto count, auto metas) {
            constexpr uint32_t COUNT = decltype(count)::value, METAS = decltype(metas)::value;
            if(T::META_WAVES == 4u || metaWave)
                r355::waitVmcnt<COUNT>();
            else
                r355::waitVmcnt<COUNT - METAS>();
        };

        // ---- LDS -> registers (per lane, fixed)
        //   block i of A (rows 16 i .. + 15 of the wave's 16 WB): 1 KiB of values in lane order, 256 B of indices
        //   block j of B: row 16 j + t, 16-byte chunks g and 4 + g of the row's 128 bytes
        const uint32_t rdA = wm * (WB * 1024u) + lane * 16u, rdM = OFF_META + (wm * (WB * 256u) + lane * 4u) / ES;
        const uint32_t rB  = wn * (16u * WB) + t, swB = (t >> 1) & 7u;
        const uint32_t rdB0 = OFF_B + rB * 128u + ((g ^ swB) * 16u), rdB1 = OFF_B + rB * 128u + (((4u + g) ^ swB) * 16u);
        uint32_t       rdBn[8] = {}; // row-major B: block j of the wave's own, first half of the lane's k-rows of K half 0
        if constexpr(!B_KCONTIG)
            r355::tile::readOffsets8<false, WB, ES>(wn, lane, rdBn);

        // piece r (0 .. 2 H - 1) of an A group: block r / 2 of the half, values (r even) or indices (r odd)
        auto readA = [&](AG& grp, uint32_t at, uint32_t half, uint32_t r) {
            const uint32_t i = H * half + (r >> 1);
            if(r & 1u)
            {
                if constexpr(ES == 1u)
                    grp.idx[r >> 1] = *reinterpret_cast<const int*>(lds + at + rdM + i * 256u);
                else
                {
                    // Only the low 16 bits are index bits (ABID 0); the high half stays undefined on purpose: widening
                    // the 16-bit value would put a VALU instruction between the LDS read and the matrix instruction,
                    // and the inline-assembly matrix instructions are invisible to the compiler's hazard handling
                    // (a VALU write directly followed by a matrix instruction that reads it delivers the old value).
                    using s16x2 = short __attribute__((ext_vector_type(2)));
                    s16x2 v;
                    v[0]            = *reinterpret_cast<const short*>(lds + at + rdM + i * 128u);
                    grp.idx[r >> 1] = __builtin_bit_cast(int, v);
                }
            }
            else
                grp.v[r >> 1] = *reinterpret_cast<const i32x4*>(lds + at + rdA + i * 1024u);
        };
        // piece r (0 .. 2 H - 1) of a B group: block r / 2 of the half, 64-byte K half r % 2 (row-major B: in two transposed parts)
        auto readB = [&](i32x8 (&grp)[H], uint32_t at, uint32_t half, uint32_t r, uint32_t part = 0u) {
            const uint32_t j = H * half + (r >> 1);
            if constexpr(B_KCONTIG)
            {
                const i32x4    v = *reinterpret_cast<const i32x4*>(lds + at + ((r & 1u) ? rdB1 : rdB0) + j * 2048u);
                const uint32_t o = 4u * (r & 1u);
                grp[r >> 1][o] = v[0], grp[r >> 1][o + 1u] = v[1], grp[r >> 1][o + 2u] = v[2], grp[r >> 1][o + 3u] = v[3];
            }
            else
                r355::tile::readBlock8<false, WB, ES>(lds + at + OFF_B, rdBn, j, r & 1u, part, grp[r >> 1], 4u * (r & 1u));
        };
        // the pieces dealt to slot n (0 .. NQ - 1) of a quadrant: a group's 2 H pieces (4 H transposed half pieces of a
        // row-major B) evenly over the NQ slots - large tile: one read per two (one) matrix instructions, small tile: one (two)
        auto readSlotA = [&](AG& grp, uint32_t at, uint32_t half, uint32_t n) {
#if !defined(R355_ABLATE_READS) && !defined(R355_SPARSE_A_DIRECT)
            constexpr uint32_t P = 2u * H;
#pragma unroll
            for(uint32_t r = (n * P + NQ - 1u) / NQ; r < ((n + 1u) * P + NQ - 1u) / NQ; ++r)
                readA(grp, at, half, r);
#endif
        };
        auto readSlotB = [&](i32x8 (&grp)[H], uint32_t at, uint32_t half, uint32_t n) {
#ifndef R355_ABLATE_READS
            constexpr uint32_t P = B_KCONTIG ? 2u * H : 4u * H;
#pragma unroll
            for(uint32_t r = (n * P + NQ - 1u) / NQ; r < ((n + 1u) * P + NQ - 1u) / NQ; ++r)
            {
                if constexpr(B_KCONTIG)
                    readB(grp, at, half, r);
                else
                    readB(grp, at, half, r >> 1, r & 1u);
            }
#endif
        };

        AccV acc[WB][WB];
#pragma unroll
        for(uint32_t i = 0; i < WB; ++i)
#pragma unroll
            for(uint32_t j = 0; j < WB; ++j)
                acc[i][j] = AccV{0, 0, 0, 0};

        AG    aLo, aHi;
        i32x8 bX[H], bY[H]; // alternate as the low / high half of B's blocks
#ifdef R355_SPARSE_A_DIRECT
        AG             aOwn[2][2]; // [stage parity][low / high four blocks]: this wave's A, requested one stage ahead
        const uint32_t aLaneV = wm * 8192u + lane * 16u, aLaneM = (wm * 2048u + lane * 4u) / ES;
        // piece n of a stage's A: 0 .. 7 the values of block n, 8 .. 15 the indices of block n - 8 (buffers that end with
        // the tile's last valid row; a stage past the end is a buffer of nothing)
        auto loadOwnA = [&](uint32_t stage, uint32_t par, uint32_t n) {
            const bool     valid = stage < numStages;
            const uint32_t st    = valid ? stage : 0u;
            if(n < 8u)
            {
                const auto rsrc = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<char*>(gA + st * strideV), 0,
                                                                    static_cast<int>(valid ? validM * 64u : 0u), 0x00020000);
                aOwn[par][n / 4u].v[n % 4u] = __builtin_bit_cast(i32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, aLaneV, n * 1024u, 0));
            }
            else
            {
                const uint32_t i    = n - 8u;
                const auto     rsrc = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<char*>(gM + st * strideM), 0,
                                                                        static_cast<int>(valid ? validM * (16u / ES) : 0u), 0x00020000);
                if constexpr(ES == 1u)
                    aOwn[par][i / 4u].idx[i % 4u] = static_cast<int>(__builtin_amdgcn_raw_buffer_load_b32(rsrc, aLaneM, i * 256u, 0));
                else
                {
                    // (low 16 bits only, the high half left undefined: see readA)
                    using s16x2 = short __attribute__((ext_vector_type(2)));
                    s16x2 v;
                    v[0]                          = __builtin_amdgcn_raw_buffer_load_b16(rsrc, aLaneM, i * 128u, 0);
                    aOwn[par][i / 4u].idx[i % 4u] = __builtin_bit_cast(int, v);
                }
            }
        };
#endif

        // load slot n of quadrant q (0: Q3, 1: Q4 of the stage that frees the slot `at`; 2: Q1, 3: Q2 of the next stage)
        auto loadSlot = [&](uint32_t q, uint32_t stage, uint32_t at, uint32_t n) {
            constexpr uint32_t COUNT[4] = {WB == 8 ? 4u : 2u, WB == 8 ? 3u : 2u, WB == 8 ? 3u : 2u, WB == 8 ? 3u : 1u};
            constexpr uint32_t STEP[4]  = {WB == 8 ? 4u : 2u, WB == 8 ? 5u : 2u, WB == 8 ? 5u : 2u, WB == 8 ? 5u : 2u};
            static_assert(COUNT[0] + COUNT[1] == T::FIRST_HALF && COUNT[0] + COUNT[1] + COUNT[2] + COUNT[3] == T::LOADS, "every load has a slot");
            uint32_t first = 0;
#pragma unroll
            for(uint32_t u = 0; u < 4; ++u)
                if(u < q)
                    first += COUNT[u];
            if(n % STEP[q] == 1u && n / STEP[q] < COUNT[q])
                issueLoad(stage, at, first + n / STEP[q]);
        };
        // (par: parity of the stage, which names the register set of the measurement build that keeps A out of LDS)
        auto stageBody = [&](uint32_t kt, uint32_t cur, uint32_t nxt, uint32_t prv, i32x8 (&bLo)[H], i32x8 (&bHi)[H], uint32_t par) {
#ifdef R355_SPARSE_A_DIRECT
            AG& aLo = aOwn[par][0];
            AG& aHi = aOwn[par][1];
#else
            (void)par;
#endif
            // Q1: A low x B low; B high arrives; the third quarter of stage kt + 2's loads (into the slot stage kt - 1 has left)
#pragma unroll
            for(uint32_t n = 0; n < NQ; ++n)
            {
                smfmac16<E>(acc[n % H][n / H], aLo.v[n % H], bLo[n / H], aLo.idx[n % H]);
                readSlotB(bHi, cur, 1, n);
#ifdef R355_SPARSE_A_DIRECT
                loadOwnA(kt + 1u, par ^ 1u, n);
#endif
                loadSlot(2u, kt + 2u, prv, n);
                __builtin_amdgcn_sched_barrier(0);
            }
            // Q2: A low x B high (column by column, in the order B arrived); A high arrives; the last of stage kt + 2's loads
#pragma unroll
            for(uint32_t n = 0; n < NQ; ++n)
            {
                smfmac16<E>(acc[n % H][H + n / H], aLo.v[n % H], bHi[n / H], aLo.idx[n % H]);
                readSlotA(aHi, cur, 1, n);
                loadSlot(3u, kt + 2u, prv, n);
                __builtin_amdgcn_sched_barrier(0);
            }
#if defined(R355_SPARSE_A_DIRECT)
            r355::waitVmcnt<8 + 16>(); // the youngest: 8 B loads of stage kt + 2 and the 16 A loads of stage kt + 1 issued under Q1
#elif defined(R355_ABLATE_LOADS)
            r355::waitVmcnt<0>();
#else
            // stage kt + 1 has landed; the youngest loads are stage kt + 2's
            waitYoungest(std::integral_constant<uint32_t, T::LOADS>{}, std::integral_constant<uint32_t, 1>{});
#endif
            r355::ldsBarrier();
            // Q3: A high x B high (row by row, in the order A arrived); next A low arrives; the first of stage kt + 3's loads
#pragma unroll
            for(uint32_t n = 0; n < NQ; ++n)
            {
                smfmac16<E>(acc[H + n / H][H + n % H], aHi.v[n / H], bHi[n % H], aHi.idx[n / H]);
                readSlotA(aLo, nxt, 0, n);
                loadSlot(0u, kt + 3u, cur, n);
                __builtin_amdgcn_sched_barrier(0);
            }
            // Q4: A high x B low; next B low arrives in the registers B high has left; the second quarter of stage kt + 3's loads
#pragma unroll
            for(uint32_t n = 0; n < NQ; ++n)
            {
                smfmac16<E>(acc[H + n % H][n / H], aHi.v[n % H], bLo[n / H], aHi.idx[n % H]);
                readSlotB(bHi, nxt, 0, n);
                loadSlot(1u, kt + 3u, cur, n);
                __builtin_amdgcn_sched_barrier(0);
            }
        };

        constexpr uint32_t SLOT[3] = {0u, STAGE_BYTES, 2u * STAGE_BYTES};
#pragma unroll
        for(uint32_t st = 0; st < RING; ++st)
#pragma unroll
            for(uint32_t x = 0; x < (st + 1u < RING ? T::LOADS : T::FIRST_HALF); ++x)
                issueLoad(st, SLOT[st], x); // (the rest of stage 2 follows under Q1 and Q2 of stage 0)
        // stage 0 has landed: stage 1 and the first half of stage 2 (an index load in each) may still be under way
        waitYoungest(std::integral_constant<uint32_t, T::LOADS + T::FIRST_HALF>{}, std::integral_constant<uint32_t, 2>{});
        r355::ldsBarrier();
#pragma unroll
        for(uint32_t r = 0; r < 2u * H; ++r)
        {
#ifndef R355_SPARSE_A_DIRECT
            readA(aLo, SLOT[0], 0, r);
#endif
            readB(bX, SLOT[0], 0, r);
            if constexpr(!B_KCONTIG)
                readB(bX, SLOT[0], 0, r, 1u);
        }
#ifdef R355_SPARSE_A_DIRECT
#pragma unroll
        for(uint32_t n = 0; n < 16; ++n)
            loadOwnA(0u, 0u, n);
#endif

        uint32_t kt = 0;
        for(uint32_t trips = numStages / 6u; trips > 0; --trips, kt += 6u)
        {
            stageBody(kt, SLOT[0], SLOT[1], SLOT[2], bX, bY, 0u);
            stageBody(kt + 1u, SLOT[1], SLOT[2], SLOT[0], bY, bX, 1u);
            stageBody(kt + 2u, SLOT[2], SLOT[0], SLOT[1], bX, bY, 0u);
            stageBody(kt + 3u, SLOT[0], SLOT[1], SLOT[2], bY, bX, 1u);
            stageBody(kt + 4u, SLOT[1], SLOT[2], SLOT[0], bX, bY, 0u);
            stageBody(kt + 5u, SLOT[2], SLOT[0], SLOT[1], bY, bX, 1u);
        }
        const uint32_t rem = numStages - kt;
        if(rem > 0u)
        {
            stageBody(kt, SLOT[0], SLOT[1], SLOT[2], bX, bY, 0u);
            if(rem > 1u)
            {
                stageBody(kt + 1u, SLOT[1], SLOT[2], SLOT[0], bY, bX, 1u);
                if(rem > 2u)
                {
                    stageBody(kt + 2u, SLOT[2], SLOT[0], SLOT[1], bX, bY, 0u);
                    if(rem > 3u)
                    {
                        stageBody(kt + 3u, SLOT[0], SLOT[1], SLOT[2], bY, bX, 1u);
                        if(rem > 4u)
                            stageBody(kt + 4u, SLOT[1], SLOT[2], SLOT[0], bX, bY, 0u);
                    }
                }
            }
        }
        // the loads past the last stage (zeros) are still landing in the slots the epilogue reuses, and the last
        // matrix instructions are still in the pipeline (the compiler knows neither)
        asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
        r355::waitVmcnt<0>();
        r355::ldsBarrier();

        // ---- epilogue.  A lane holds D(16 i + 4 g + e, 16 j + t), e = 0..3, of each block: four consecutive
        // rows of one column.
        // (the lane number is taken afresh - ordered after the K loop's matrix instructions - so that nothing derived from
        // it for the epilogue occupies a register, or a spill slot, during the K loop)
        uint32_t laneE;
        asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(laneE));
        const uint32_t tE = laneE & 15u, gE = laneE >> 4;
        const AccE     alpha = static_cast<AccE>(p.alpha), beta = static_cast<AccE>(p.beta);
        const uint32_t m0 = tm * T::M + wm * (16u * WB), n0 = tn * T::N + wn * (16u * WB);
        using V4 = AccE __attribute__((ext_vector_type(4)));
        if(!p.dRow)
        {
            // col-major: a lane's four rows are contiguous
#pragma unroll
            for(uint32_t i = 0; i < WB; ++i)
#pragma unroll
                for(uint32_t j = 0; j < WB; ++j)
                {
                    const uint32_t row = m0 + 16u * i + 4u * gE, col = n0 + 16u * j + tE;
                    if(row >= p.m || col >= p.n) // (m is a multiple of 16: a lane's four rows are inside or outside together)
                        continue;
                    V4             out;
#pragma unroll
                    for(uint32_t e = 0; e < 4; ++e)
                        out[e] = alpha * acc[i][j][e];
                    if(beta != static_cast<AccE>(0))
                    {
                        const V4 cv = *reinterpret_cast<const V4*>(p.c + ((uint64_t)col * p.ldc + row) * 4u);
#pragma unroll
                        for(uint32_t e = 0; e < 4; ++e)
                            out[e] += beta * cv[e];
                    }
                    *reinterpret_cast<V4*>(p.d + ((uint64_t)col * p.ldd + row) * 4u) = out;
                }
            return;
        }
        // row-major: transpose through this wave's quarter of the idle stage slots, 64 rows (four block rows) at a time:
        // rows of 16 WB x 4 bytes = CH chunks of 16 bytes, chunk c of row r in slot c ^ (r % CH) -- the 64 lanes of a write
        // (rows 4 g + e, columns 16 j + t) and of a read (64 / CH whole rows) each cover all 64 banks once.
        constexpr uint32_t CH = 4u * WB, ROW_BYTES = 64u * WB, PASSES = WB / 4u;
        char*              wl = lds + wave * (RING * STAGE_BYTES / 4u);
        static_assert(RING * STAGE_BYTES / 4u >= 64u * ROW_BYTES, "a wave's share of LDS holds 64 rows of its tile");
#pragma unroll
        for(uint32_t pass = 0; pass < PASSES; ++pass)
        {
#pragma unroll
            for(uint32_t ii = 0; ii < 4; ++ii)
#pragma unroll
                for(uint32_t j = 0; j < WB; ++j)
#pragma unroll
                    for(uint32_t e = 0; e < 4; ++e)
                    {
                        const uint32_t row = 16u * ii + 4u * gE + e, col = 16u * j + tE;
                        *reinterpret_cast<AccE*>(wl + row * ROW_BYTES + (((col >> 2) ^ (row & (CH - 1u))) * 16u) + (col & 3u) * 4u)
                            = alpha * acc[4u * pass + ii][j][e];
                    }
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for(uint32_t it = 0; it < CH; ++it)
            {
                const uint32_t L = it * 64u + laneE, row = L / CH, c = L % CH;
                V4             v = *reinterpret_cast<const V4*>(wl + row * ROW_BYTES + ((c ^ (row & (CH - 1u))) * 16u));
                const uint64_t off = (uint64_t)(m0 + 64u * pass + row);
                if(off >= p.m || n0 + 4u * c >= p.n) // (n is a multiple of 16: a 16-byte chunk is inside or outside D as a whole)
                    continue;
                if(beta != static_cast<AccE>(0))
                {
                    const V4 cv = *reinterpret_cast<const V4*>(p.c + (off * p.ldc + n0) * 4u + c * 16u);
#pragma unroll
                    for(uint32_t e = 0; e < 4; ++e)
                        v[e] += beta * cv[e];
                }
                __builtin_nontemporal_store(v, reinterpret_cast<V4*>(p.d + (off * p.ldd + n0) * 4u + c * 16u));
            }
            __builtin_amdgcn_wave_barrier();
        }
    }

    // (a waves-per-EU attribute that depends on a template parameter makes the compiler drop the host-side launch stub:
    // one __global__ wrapper per tile size)
    template <SpElem E, bool B_KCONTIG>
    __global__ void __launch_bounds__(T_THREADS) __attribute__((amdgpu_waves_per_eu(1, 1))) sparseTiledKernel(TiledParams p)
    {
        sparseTiled<E, B_KCONTIG, 8>(p);
    }
#ifndef R355_SPARSE_A_DIRECT
    template <SpElem E, bool B_KCONTIG>
    __global__ void __launch_bounds__(T_THREADS) sparseTiledKernelSmall(TiledParams p)
    {
        sparseTiled<E, B_KCONTIG, 4>(p);
    }
#endif

    // The macro tiles run any m, n (multiples of 16) and k (whole stages); under AUTO they are taken from 128 x 128 on
    // (below that most of a tile's matrix instructions would multiply padding).
    bool tiledOk(const r355_gemm_args& g)
    {
        const uint32_t es = (g.in_type == R355_F16 || g.in_type == R355_BF16) ? 2u : 1u;
        const bool     forced = g.kernel == R355_KERNEL_TILED || g.kernel == R355_KERNEL_TILED_DEEP || g.kernel == R355_KERNEL_TILED_128;
        const bool     shape  = forced || (g.m >= 128u && g.n >= 128u);
        return g.kernel != R355_KERNEL_SIMPLE && shape && (g.beta == 0.0 || g.layout_c == g.layout_d) && r355::aligned(g.a_meta, 16)
               && (uint64_t)g.ldb * es <= (1u << 23);
    }

    // Macro tile edge, from a timing model of a launch: rounds over the CUs - one large tile or two small ones per CU and
    // round - each costing a fixed part plus a part per 128-byte stage of K.  Microseconds, fitted to 8-bit launches of
    // 1024^2 ... 8192^2 with k from 512 to 8192 (the 16-bit kernels move the same bytes per stage):
    //                                        fixed   per stage
    //   256 x 256, every CU busy           15 / 18    0.79      (first / later rounds) the K loop is bound by what the L2 delivers
    //   256 x 256, at most half the CUs    15 / 18    0.48      to all CUs at once; with half of them idle, by its matrix instructions
    //   128 x 128, two on every CU            5.4     0.635     (half the work of a large round)
    //   128 x 128, one on every CU            3.5     0.365
    //   128 x 128, one on a few CUs           3.5     0.28
    // and linear in the number of tiles of the last round in between.  So the small tile wins where the large tiles would
    // leave CUs idle (2048^2 x 8192: 26 us against 48) and, with all CUs busy, up to about 12 stages, where the large
    // tile's prologue and epilogue - which nothing overlaps with one workgroup per CU - weigh as much as its K loop
    // (8192^2 x 1024: 81 us against 97); the large tile is 1.35 times faster on long K with the chip full.
    uint32_t macroTile(const r355_gemm_args& g)
    {
#ifdef R355_SPARSE_A_DIRECT
        return 256u;
#endif
        if(g.kernel == R355_KERNEL_TILED || g.kernel == R355_KERNEL_TILED_DEEP)
            return 256u; // (DEEP: one and the same here)
        if(g.kernel == R355_KERNEL_TILED_128)
            return 128u;
        const uint32_t es     = (g.in_type == R355_F16 || g.in_type == R355_BF16) ? 2u : 1u;
        const double   stages = static_cast<double>((uint64_t)g.k * es / T_K);
        const uint64_t cus    = r355::computeUnits();
        const uint64_t t256   = (uint64_t)((g.m + 255u) / 256u) * ((g.n + 255u) / 256u);
        const uint64_t t128   = (uint64_t)((g.m + 127u) / 128u) * ((g.n + 127u) / 128u);
        const double   perCu  = 1.0 / static_cast<double>(cus);
        double         cost256 = static_cast<double>(t256 / cus) * (18.0 + 0.79 * stages) - 3.0;
        if(const uint64_t rest = t256 % cus)
        {
            const double over = 2.0 * static_cast<double>(rest) * perCu - 1.0; // 0 at half of the CUs, 1 at all of them
            cost256 += 18.0 + stages * (0.48 + 0.31 * (over > 0.0 ? over : 0.0));
        }
        double cost128 = static_cast<double>(t128 / (2u * cus)) * (5.4 + 0.635 * stages);
        if(const uint64_t rest = t128 % (2u * cus))
        {
            const double f = static_cast<double>(rest) * perCu; // tiles per CU: 0 .. 2
            cost128 += f <= 1.0 ? 3.5 + stages * (0.28 + 0.085 * f) : 3.5 + 1.9 * (f - 1.0) + stages * (0.365 + 0.27 * (f - 1.0));
        }
        return cost128 * 1.02 < cost256 ? 128u : 256u; // (over 156 measured shapes the slower tile 6 times, by 2.6 % at most)
    }

    uint32_t simpleBlock(const r355_gemm_args& g)
    {
        return (g.m % 32u == 0u && g.n % 32u == 0u) ? 32u : 16u;
    }
} // namespace

namespace r355
{
    int gemmSparseCheck(const r355_gemm_args& g, r355_gemm_plan* plan)
    {
        const bool i8 = g.in_type == R355_I8 && g.out_type == R355_I32;
        const bool f8 = g.in_type == R355_E4M3 && g.out_type == R355_F32;
        const bool w  = (g.in_type == R355_F16 || g.in_type == R355_BF16) && g.out_type == R355_F32;
        if(!i8 && !f8 && !w)
            return fail(R355_ERR_UNSUPPORTED, "sparse gemm: supported types are i8 -> i32 and e4m3 | f16 | bf16 -> f32");
        if(g.layout_a != R355_ROW_MAJOR)
            return fail(R355_ERR_UNSUPPORTED, "sparse gemm: compressed A is K-blocked row storage (R355_ROW_MAJOR)");
        if(!g.a_meta)
            return fail(R355_ERR_BAD_ARG, "sparse gemm: a_meta is null");
        const uint32_t es = w ? 2u : 1u, kStage = 128u / es; // element bytes, dense k per stage of the storage format
        if(g.m % 16 || g.n % 16 || g.k % kStage)
            return fail(R355_ERR_BAD_SIZE, "sparse gemm: m=%u n=%u must be multiples of 16 and k=%u of %u", g.m, g.n, g.k, kStage);
        if(g.lda != g.k / 2u)
            return fail(R355_ERR_BAD_ARG, "sparse gemm: the K-blocked storage of A has no padding: lda=%u must be k / 2 = %u", g.lda, g.k / 2u);
        if(!aligned(g.a, 16) || !aligned(g.b, 16) || (g.ldb * es) % 16 || !aligned(g.a_meta, 4) || !aligned(g.d, 16) || (g.ldd % 4)
           || (g.beta != 0.0 && (!aligned(g.c, 16) || (g.ldc % 4))))
            return fail(R355_ERR_MISALIGNED, "sparse gemm: values, B, C and D need 16-byte alignment (pointers and leading dimensions), metadata 4-byte");
        if(g.kernel == R355_KERNEL_TILED_128_SPLITK)
            return fail(R355_ERR_UNSUPPORTED, "sparse gemm: no split along K (R355_KERNEL_TILED_128 is the 128 x 128 macro tile)");
        if((g.kernel == R355_KERNEL_TILED || g.kernel == R355_KERNEL_TILED_DEEP || g.kernel == R355_KERNEL_TILED_128) && !tiledOk(g))
            return fail(R355_ERR_UNSUPPORTED,
                        "sparse gemm (macro tile): C (when beta != 0) and D must share an orientation, metadata 16-byte aligned, ldb below 8 MiB");
        if(plan && tiledOk(g))
        {
            const uint32_t tile = macroTile(g);
            plan->kernel       = tile == 256u ? R355_KERNEL_TILED : R355_KERNEL_TILED_128;
            plan->macro_tile_m = tile;
            plan->macro_tile_n = tile;
            plan->macro_tile_k = T_K / es;
            plan->grid_x       = ((((g.m + tile - 1) / tile) * ((g.n + tile - 1) / tile) + 7u) / 8u) * 8u;
            plan->grid_y       = 1;
            plan->block_x      = T_THREADS;
            plan->block_y      = 1;
            plan->lds_bytes    = RING * (tile == 256u ? SpTile<8>::STAGE_BYTES : SpTile<4>::STAGE_BYTES);
        }
        else if(plan)
        {
            const uint32_t blk = simpleBlock(g);
            plan->kernel       = R355_KERNEL_SIMPLE;
            plan->macro_tile_m = blk * WAVES_X;
            plan->macro_tile_n = blk * WAVES_Y;
            plan->macro_tile_k = kStage;
            plan->grid_x       = (g.m + blk * WAVES_X - 1) / (blk * WAVES_X);
            plan->grid_y       = (g.n + blk * WAVES_Y - 1) / (blk * WAVES_Y);
            plan->block_x      = WAVES_X * 64;
            plan->block_y      = WAVES_Y;
            plan->lds_bytes    = 0;
        }
        return R355_OK;
    }

    template <typename InT, typename AccE>
    static int launchSimple(const r355_gemm_args& g, hipStream_t stream)
    {
        const uint32_t blk = simpleBlock(g);
        dim3           block(WAVES_X * 64, WAVES_Y);
        dim3           grid((g.m + blk * WAVES_X - 1) / (blk * WAVES_X), (g.n + blk * WAVES_Y - 1) / (blk * WAVES_Y));
        const layout_t lb = g.layout_b == R355_ROW_MAJOR ? mem_row_major : mem_col_major;
        const layout_t lc = g.layout_c == R355_ROW_MAJOR ? mem_row_major : mem_col_major;
        const layout_t ld = g.layout_d == R355_ROW_MAJOR ? mem_row_major : mem_col_major;
        auto           go = [&](auto kernel) {
            hipLaunchKernelGGL(kernel, grid, block, 0, stream, g.m, g.n, g.k, static_cast<const InT*>(g.a),
                               static_cast<const uint8_t*>(g.a_meta), static_cast<const InT*>(g.b), static_cast<const AccE*>(g.c),
                               static_cast<AccE*>(g.d), g.ldb, g.ldc, g.ldd, lb, lc, ld, static_cast<AccE>(g.alpha), static_cast<AccE>(g.beta));
        };
        if(blk == 32u)
            go(sparseBlockPerWave<InT, AccE, 32>);
        else
            go(sparseBlockPerWave<InT, AccE, 16>);
        return checkLaunch("sparse gemm");
    }

    int gemmSparseLaunch(const r355_gemm_args& g, hipStream_t stream)
    {
        if(tiledOk(g))
        {
            TiledParams p;
            p.m = g.m, p.n = g.n, p.k = g.k;
            p.aVals = static_cast<const uint8_t*>(g.a), p.aMeta = static_cast<const uint8_t*>(g.a_meta);
            p.b = static_cast<const uint8_t*>(g.b);
            p.c = static_cast<const char*>(g.c), p.d = static_cast<char*>(g.d);
            p.ldb = g.ldb, p.ldc = g.ldc, p.ldd = g.ldd;
            p.alpha = g.alpha, p.beta = g.beta;
            const uint32_t tile = macroTile(g);
            p.tilesM = (g.m + tile - 1) / tile, p.tilesN = (g.n + tile - 1) / tile;
            p.dRow = g.layout_d == R355_ROW_MAJOR;
            const dim3 grid(((p.tilesM * p.tilesN + 7u) / 8u) * 8u), block(T_THREADS);
            auto go = [&](auto bk, auto large) {
                constexpr bool BK = decltype(bk)::value;
                auto           launch = [&](auto elem) {
                    constexpr SpElem E = decltype(elem)::value;
#ifndef R355_SPARSE_A_DIRECT
                    if constexpr(!decltype(large)::value)
                        hipLaunchKernelGGL((sparseTiledKernelSmall<E, BK>), grid, block, 0, stream, p);
                    else
#endif
                        hipLaunchKernelGGL((sparseTiledKernel<E, BK>), grid, block, 0, stream, p);
                };
                switch(g.in_type)
                {
                case R355_E4M3: launch(std::integral_constant<SpElem, SpElem::E4M3>{}); break;
                case R355_F16: launch(std::integral_constant<SpElem, SpElem::F16>{}); break;
                case R355_BF16: launch(std::integral_constant<SpElem, SpElem::BF16>{}); break;
                default: launch(std::integral_constant<SpElem, SpElem::I8>{}); break;
                }
            };
            const bool colB = g.layout_b == R355_COL_MAJOR;
            if(tile == 256u)
                colB ? go(std::true_type{}, std::true_type{}) : go(std::false_type{}, std::true_type{});
            else
                colB ? go(std::true_type{}, std::false_type{}) : go(std::false_type{}, std::false_type{});
            return checkLaunch("sparse gemm (macro tile)");
        }
        switch(g.in_type)
        {
        case R355_E4M3: return launchSimple<float8_t, float>(g, stream);
        case R355_F16: return launchSimple<float16_t, float>(g, stream);
        case R355_BF16: return launchSimple<bfloat16_t, float>(g, stream);
        default: return launchSimple<int8_t, int32_t>(g, stream);
        }
    }
} // namespace r355

namespace
{
    // Byte offsets of (row, dense group of four `grp`) in the K-blocked storage: the group's two kept elements and
    // its index nibble.  A stage holds 32 / ES groups of a row, a lane group 8 / ES of them.
    template <typename T>
    struct Place
    {
        size_t   value; // element index of the first kept element
        size_t   metaByte;
        uint32_t metaShift;
    };
    template <typename T>
    Place<T> placeOf(uint32_t row, uint32_t grp, uint32_t m)
    {
        using S                  = rocwmma::Sparse24<T>;
        constexpr uint32_t perLg = S::ChunkElems / 2u; // groups per lane group: 8 (1-byte) or 4 (2-byte elements)
        const uint32_t stage = grp / (4u * perLg), lg = (grp / perLg) % 4u, within = grp % perLg;
        Place<T>       pl;
        pl.value = (size_t)stage * S::valueStageStride(m) + S::valueByteInStage(row, lg) / sizeof(T) + 2u * within;
        pl.metaByte  = (size_t)stage * S::metaStageStride(m) + S::metaByteInStage(row, lg) + within / 2u;
        pl.metaShift = 4u * (within & 1u);
        return pl;
    }

    // An element counts as zero when all its bits are zero (a kept -0.0 stays a kept value: the round trip is exact).
    template <typename T>
    int compress24(const T* dense, uint32_t m, uint32_t k, T* values, uint8_t* meta)
    {
        if(!dense || !values || !meta)
            return r355::fail(R355_ERR_BAD_ARG, "compress_24: null pointer");
        if(m % 16u || k % rocwmma::Sparse24<T>::StageK)
            return r355::fail(R355_ERR_BAD_SIZE, "compress_24: m=%u must be a multiple of 16 and k=%u of %u", m, k,
                              rocwmma::Sparse24<T>::StageK);
        memset(meta, 0, (size_t)m * k / 8u);
        for(uint32_t r = 0; r < m; ++r)
        {
            const T* src = dense + (size_t)r * k;
            for(uint32_t g = 0; g < k / 4u; ++g)
            {
                // positions of the kept pair: the non-zeros first, then the lowest free positions
                uint32_t keep = 0, count = 0; // bit mask over the 4 positions
                for(uint32_t e = 0; e < 4; ++e)
                    if(src[4 * g + e] != 0)
                        keep |= 1u << e, ++count;
                if(count > 2)
                    return r355::fail(R355_ERR_NOT_24_SPARSE, "compress_24: row %u, group %u holds %u non-zeros", r, g, count);
                for(uint32_t e = 0; e < 4 && count < 2; ++e)
                    if(!(keep & (1u << e)))
                        keep |= 1u << e, ++count;
                uint32_t pos[2], p = 0;
                for(uint32_t e = 0; e < 4; ++e)
                    if(keep & (1u << e))
                        pos[p++] = e;
                const Place<T> pl    = placeOf<T>(r, g, m);
                values[pl.value]     = src[4 * g + pos[0]];
                values[pl.value + 1] = src[4 * g + pos[1]];
                meta[pl.metaByte] |= static_cast<uint8_t>((pos[0] | (pos[1] << 2)) << pl.metaShift);
            }
        }
        return R355_OK;
    }

    template <typename T>
    int decompress24(const T* values, const uint8_t* meta, uint32_t m, uint32_t k, T* dense)
    {
        if(!dense || !values || !meta)
            return r355::fail(R355_ERR_BAD_ARG, "decompress_24: null pointer");
        if(m % 16u || k % rocwmma::Sparse24<T>::StageK)
            return r355::fail(R355_ERR_BAD_SIZE, "decompress_24: m=%u must be a multiple of 16 and k=%u of %u", m, k,
                              rocwmma::Sparse24<T>::StageK);
        memset(dense, 0, (size_t)m * k * sizeof(T));
        for(uint32_t r = 0; r < m; ++r)
            for(uint32_t g = 0; g < k / 4u; ++g)
            {
                const Place<T> pl  = placeOf<T>(r, g, m);
                const uint32_t nib = (meta[pl.metaByte] >> pl.metaShift) & 0xFu;
                dense[(size_t)r * k + 4 * g + (nib & 3u)]  = values[pl.value];
                dense[(size_t)r * k + 4 * g + (nib >> 2)] = values[pl.value + 1];
            }
        return R355_OK;
    }
} // namespace

extern "C" int r355_compress_24(const uint8_t* dense, uint32_t m, uint32_t k, uint8_t* values, uint8_t* meta)
{
    return compress24(dense, m, k, values, meta);
}

extern "C" int r355_decompress_24(const uint8_t* values, const uint8_t* meta, uint32_t m, uint32_t k, uint8_t* dense)
{
    return decompress24(values, meta, m, k, dense);
}

extern "C" int r355_compress_24_16(const uint16_t* dense, uint32_t m, uint32_t k, uint16_t* values, uint8_t* meta)
{
    return compress24(dense, m, k, values, meta);
}

extern "C" int r355_decompress_24_16(const uint16_t* values, const uint8_t* meta, uint32_t m, uint32_t k, uint16_t* dense)
{
    return decompress24(values, meta, m, k, dense);
}
