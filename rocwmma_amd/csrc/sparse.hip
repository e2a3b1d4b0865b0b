// 2:4 structured-sparse GEMM on gfx950 sparse matrix cores (v_smfmac_*), plus the host-side
// compressor.  The reference has no sparse path; the storage format is defined here.
//
// A (m x k, row-major; 1-byte elements, or f16 / bf16 for the block-per-wave kernel) keeps 2 of every aligned
// group of 4 along k:
//   values  m x k/2   the kept pair of each group, in position order
//   meta    m x k/8   one nibble per group = idx0 | idx1 << 2 (idx0 < idx1), even group in the
//                     low nibble -- 32 bits cover 32 dense k, which is exactly the index
//                     register one lane feeds to v_smfmac_*_32x32x64 for its 16 kept values.
// B is dense, col-major (k contiguous); D row- or col-major.
//
// Two kernels:
//   sparseTiledKernel    256 x 256 macro tile, 128 dense K per stage, a ring of three LDS slots filled
//                        by direct-to-LDS loads two stages ahead (kept values 16 KiB + indices 4 KiB
//                        + dense B 32 KiB per stage), 2 x 2 waves with 4 x 4 v_smfmac_*_32x32x64
//                        accumulators each; the result is transposed through LDS so that D leaves in
//                        whole rows.
//   sparseBlockPerWave   one 32 x 32 block of D per wave straight from global memory; fallback
//                        for shapes that do not fill a macro tile.
// Per 64-wide K step a lane feeds 16 kept bytes + 4 index bytes of A and 2 x 16 dense bytes of B.  Operand formats of v_smfmac_*_32x32x64 as measured on MI355X: index
// bits [2 p + 1 : 2 p] give the position within its group of 4 of kept byte p of the lane.
// 16-bit elements run v_smfmac_f32_32x32x32_{f16,bf16}: 8 kept values + 16 index bits (the half of the index
// register that ABID names) of A and 2 x 8 dense values of B per lane and 32-wide K step, same pairing of lane
// groups, same index bits (measured with one-hot A against coded B).
#include <hip/hip_runtime.h>

#include <cstring>

#include "common.hpp"
#include "lds_dma.hpp"
#include "tile_map.hpp"

namespace
{
    using i32x4  = int __attribute__((ext_vector_type(4)));
    using i32x8  = int __attribute__((ext_vector_type(8)));
    using i32x16 = int __attribute__((ext_vector_type(16)));
    using f32x16 = float __attribute__((ext_vector_type(16)));
    using f16x8   = _Float16 __attribute__((ext_vector_type(8)));
    using f16x16  = _Float16 __attribute__((ext_vector_type(16)));
    using bf16x8  = __bf16 __attribute__((ext_vector_type(8)));
    using bf16x16 = __bf16 __attribute__((ext_vector_type(16)));

    constexpr uint32_t WAVES_X = 2, WAVES_Y = 2;

    enum class SpElem
    {
        I8,
        E4M3,
        F16,
        BF16
    };

    template <SpElem E>
    __global__ void __launch_bounds__(WAVES_X* WAVES_Y * 64) sparseBlockPerWave(uint32_t       m,
                                                                               uint32_t       n,
                                                                               uint32_t       k,
                                                                               const uint8_t* aVals,
                                                                               const uint8_t* aMeta,
                                                                               const uint8_t* b,
                                                                               const void*    c,
                                                                               void*          d,
                                                                               uint32_t       lda, // compressed values per row
                                                                               uint32_t       ldb,
                                                                               uint32_t       ldc,
                                                                               uint32_t       ldd,
                                                                               bool           cRow,
                                                                               bool           dRow,
                                                                               double         alphaF,
                                                                               double         betaF)
    {
        constexpr bool     WIDE = E == SpElem::F16 || E == SpElem::BF16; // 2-byte elements
        constexpr uint32_t ES = WIDE ? 2u : 1u, KSTEP = WIDE ? 32u : 64u; // dense k per instruction
        using Acc  = std::conditional_t<E == SpElem::I8, i32x16, f32x16>;
        using AccE = std::conditional_t<E == SpElem::I8, int, float>;
        const uint32_t lane = threadIdx.x & 63u;
        const uint32_t row0 = (blockIdx.x * WAVES_X + threadIdx.x / 64u) * 32u;
        const uint32_t col0 = (blockIdx.y * WAVES_Y + threadIdx.y) * 32u;
        if(row0 >= m || col0 >= n)
            return;
        const uint32_t idx = lane & 31u, g = lane >> 5;

        // byte pointers; a lane moves 16 bytes of kept values, KSTEP / 16 index bytes and 2 x 16 bytes of B per step
        const uint8_t* pa = aVals + ((uint64_t)(row0 + idx) * lda) * ES + 16u * g;
        const uint8_t* pm = aMeta + (uint64_t)(row0 + idx) * (k / 8u) + (KSTEP / 16u) * g;
        // The instruction pairs A's lane group g, kept bytes [8 q, 8 q + 8) with B's lane group q,
        // dense bytes [16 g, 16 g + 16).  With A's lane group g holding the kept values of dense
        // k in [32 g, 32 g + 32), B's lane group h therefore holds dense k in [16 h, 16 h + 16)
        // and [32 + 16 h, 48 + 16 h) of each 64-wide step (16-bit elements: the same in units of
        // 2 bytes, a 32-wide step).
        const uint8_t* pb = b + ((uint64_t)(col0 + idx) * ldb) * ES + 16u * g;

        Acc acc;
#pragma unroll
        for(uint32_t e = 0; e < 16; ++e)
            acc[e] = 0;

        for(uint32_t kd = 0; kd < k; kd += KSTEP)
        {
            const i32x4 av = *reinterpret_cast<const i32x4*>(pa + (kd / 2u) * ES);
            const i32x4 b0 = *reinterpret_cast<const i32x4*>(pb + kd * ES);
            const i32x4 b1 = *reinterpret_cast<const i32x4*>(pb + kd * ES + 32u);
            const i32x8 bv = {b0[0], b0[1], b0[2], b0[3], b1[0], b1[1], b1[2], b1[3]};
            if constexpr(WIDE)
            {
                const int meta = *reinterpret_cast<const uint16_t*>(pm + kd / 8u); // low half, ABID 0
                if constexpr(E == SpElem::F16)
                    acc = __builtin_amdgcn_smfmac_f32_32x32x32_f16(__builtin_bit_cast(f16x8, av),
                                                                   __builtin_bit_cast(f16x16, bv), acc, meta, 0, 0);
                else
                    acc = __builtin_amdgcn_smfmac_f32_32x32x32_bf16(__builtin_bit_cast(bf16x8, av),
                                                                    __builtin_bit_cast(bf16x16, bv), acc, meta, 0, 0);
            }
            else
            {
                const int meta = *reinterpret_cast<const int*>(pm + kd / 8u);
                if constexpr(E == SpElem::E4M3)
                    acc = __builtin_amdgcn_smfmac_f32_32x32x64_fp8_fp8(av, bv, acc, meta, 0, 0);
                else
                    acc = __builtin_amdgcn_smfmac_i32_32x32x64_i8(av, bv, acc, meta, 0, 0);
            }
        }

        // lane holds D(row0 + 8 (e / 4) + 4 g + e % 4, col0 + idx)
        const AccE alpha = static_cast<AccE>(alphaF), beta = static_cast<AccE>(betaF);
#pragma unroll
        for(uint32_t e = 0; e < 16; ++e)
        {
            const uint32_t r  = row0 + 8u * (e >> 2) + 4u * g + (e & 3u);
            const uint32_t cc = col0 + idx;
            AccE           v  = alpha * acc[e];
            if(beta != static_cast<AccE>(0))
                v += beta * static_cast<const AccE*>(c)[cRow ? (uint64_t)r * ldc + cc : (uint64_t)cc * ldc + r];
            static_cast<AccE*>(d)[dRow ? (uint64_t)r * ldd + cc : (uint64_t)cc * ldd + r] = v;
        }
    }

    // ------------------------------------------------------------------ macro-tile kernel
    constexpr uint32_t T_M = 256, T_N = 256, T_K = 128; // dense K per stage
    constexpr uint32_t T_THREADS   = 256;
    constexpr uint32_t A_BYTES     = T_M * (T_K / 2); // 16 KiB kept values
    constexpr uint32_t META_BYTES  = T_M * (T_K / 8); // 4 KiB indices
    constexpr uint32_t B_BYTES     = T_N * T_K; // 32 KiB dense
    constexpr uint32_t OFF_META    = A_BYTES;
    constexpr uint32_t OFF_B       = A_BYTES + META_BYTES;
    constexpr uint32_t STAGE_BYTES = A_BYTES + META_BYTES + B_BYTES; // 52 KiB

    struct TiledParams
    {
        uint32_t       m, n, k;
        const uint8_t* aVals;
        const uint8_t* aMeta;
        const uint8_t* b;
        const char*    c;
        char*          d;
        uint32_t       lda, ldb, ldc, ldd;
        double         alpha, beta;
        uint32_t       tilesM, tilesN;
        uint32_t       dRow; // D (and C) row-major
    };

    // Three 52 KiB stage slots (156 of 160 KiB): a stage's 32 matrix instructions last about as long
    // as half the latency of a direct load, so the slot of stage kt is refilled with stage kt + 3 and
    // two stages of loads (104 KiB per CU) are in flight at any time.  The direct loads are explicit
    // (lds_dma.hpp) and the only vmcnt wait is "all but the youngest 13" before each barrier; loads
    // past the last stage are clamped to it, so every stage issues the same 13.  Every matrix
    // instruction is followed by one LDS read and (second half of a stage) one direct load, pinned
    // by scheduling barriers.  Three stages bring every slot back to its role: single-exit loop of
    // three plus up to two stages of straight-line code.
    constexpr uint32_t RING = 3, LOADS_PER_STAGE = 13;

    template <bool FP8>
    __global__ void __launch_bounds__(T_THREADS) __attribute__((amdgpu_waves_per_eu(1, 1)))
        sparseTiledKernel(TiledParams p)
    {
        using Acc  = std::conditional_t<FP8, f32x16, i32x16>;
        using AccE = std::conditional_t<FP8, float, int>;
        using r355::loadToLds;

        __shared__ __attribute__((aligned(1024))) char lds[RING * STAGE_BYTES];

        uint32_t tm, tn;
        if(!r355::tileCoord(blockIdx.x, p.tilesM, p.tilesN, tm, tn))
            return;

        const uint32_t tid  = threadIdx.x;
        const uint32_t lane = tid & 63u;
        const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const uint32_t wm = wave >> 1, wn = wave & 1u;
        const uint32_t r32 = lane & 31u, g = lane >> 5;
        const uint32_t ldsBase
            = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) char*)lds));

        // ---- global -> LDS (per thread, fixed).  LDS chunk L = j * 256 + tid of each operand tile.
        //   kept values: 4 chunks per row, chunk c of row r in slot c ^ ((r >> 2) & 3)
        //   dense B:     8 chunks per row, chunk c of row r in slot c ^ ((r >> 1) & 7)
        //   indices:     one 16-byte chunk per row, thread t <-> row t
        const uint32_t rowA = tid >> 2, slotA = tid & 3u;
        const uint32_t gOffA = rowA * p.lda + ((slotA ^ ((rowA >> 2) & 3u)) * 16u), gStepA = 64u * p.lda;
        const uint32_t rowB = tid >> 3, slotB = tid & 7u;
        const uint32_t gOffB = rowB * p.ldb + ((slotB ^ ((rowB >> 1) & 7u)) * 16u), gStepB = 32u * p.ldb;
        const uint32_t gOffM = tid * (p.k / 8u);
        const uint32_t numStages = p.k / T_K;
        const uint64_t gA = r355::uniformAddress(p.aVals + (uint64_t)tm * T_M * p.lda);
        const uint64_t gM = r355::uniformAddress(p.aMeta + (uint64_t)tm * T_M * (p.k / 8u));
        const uint64_t gB = r355::uniformAddress(p.b + (uint64_t)tn * T_N * p.ldb);
        const uint32_t dmaDst = ldsBase + wave * 1024u; // lane l lands at dmaDst + slot + piece + 16 l

        // load x (0..12) of stage `stage` (already clamped) into the slot at byte `at`
        auto issueLoad = [&](uint32_t stage, uint32_t at, uint32_t x) {
            if(x < 4u) // 64 rows of kept values per load
                loadToLds(r355::rawBuffer(gA + stage * (T_K / 2u)), gOffA, x * gStepA, dmaDst + at + x * 4096u);
            else if(x == 4u)
                loadToLds(r355::rawBuffer(gM + stage * (T_K / 8u)), gOffM, 0u, dmaDst + at + OFF_META);
            else // 32 rows of B per load
                loadToLds(r355::rawBuffer(gB + stage * T_K), gOffB, (x - 5u) * gStepB, dmaDst + at + OFF_B + (x - 5u) * 4096u);
        };
        auto clampStage = [&](uint32_t stage) { return stage < numStages ? stage : numStages - 1u; };

        // ---- LDS -> registers (per lane, fixed)
        const uint32_t rA   = wm * 128u + r32, rB = wn * 128u + r32;
        const uint32_t swA  = (r32 >> 2) & 3u, swB = (r32 >> 1) & 7u;
        uint32_t       rdA[2], rdB[4];
#pragma unroll
        for(uint32_t q = 0; q < 2; ++q) // K group q: kept-value chunk 2 q + g
            rdA[q] = rA * 64u + (((2u * q + g) ^ swA) * 16u);
        const uint32_t rdM = OFF_META + rA * 16u + 4u * g; // + 8 q
#pragma unroll
        for(uint32_t s = 0; s < 4; ++s) // K group q uses dense chunks 4 q + g and 4 q + 2 + g
            rdB[s] = OFF_B + rB * 128u + (((2u * s + g) ^ swB) * 16u);

        struct Frags
        {
            i32x4 a[4];
            int   idx[4];
            i32x4 b0[4], b1[4];
        };
        // read x (0..15) of K group q: the four operands of block index x / 4, values first
        auto readPiece = [&](Frags& f, uint32_t at, uint32_t q, uint32_t x) {
            const uint32_t i = x >> 2;
            const char*    base = lds + at;
            switch(x & 3u)
            {
            case 0: f.a[i] = *reinterpret_cast<const i32x4*>(base + rdA[q] + i * 32u * 64u); break;
            case 1: f.idx[i] = *reinterpret_cast<const int*>(base + rdM + 8u * q + i * 32u * 16u); break;
            case 2: f.b0[i] = *reinterpret_cast<const i32x4*>(base + rdB[2u * q] + i * 32u * 128u); break;
            default: f.b1[i] = *reinterpret_cast<const i32x4*>(base + rdB[2u * q + 1u] + i * 32u * 128u); break;
            }
        };

        Acc acc[4][4];
#pragma unroll
        for(uint32_t i = 0; i < 4; ++i)
#pragma unroll
            for(uint32_t j = 0; j < 4; ++j)
#pragma unroll
                for(uint32_t e = 0; e < 16; ++e)
                    acc[i][j][e] = 0;

        // matrix instruction n (0..15) of a K group: L-shaped shells, so that block index d of either
        // operand is first needed after d * d instructions (the reads arrive block by block)
        auto mfmaAt = [&](const Frags& f, uint32_t n) {
            uint32_t d = 0;
            while((d + 1u) * (d + 1u) <= n)
                ++d;
            const uint32_t r = n - d * d;
            const uint32_t i = r <= d ? d : r - d - 1u, j = r <= d ? r : d;
            const i32x8    bv = {f.b0[j][0], f.b0[j][1], f.b0[j][2], f.b0[j][3], f.b1[j][0], f.b1[j][1], f.b1[j][2], f.b1[j][3]};
            if constexpr(FP8)
                acc[i][j] = __builtin_amdgcn_smfmac_f32_32x32x64_fp8_fp8(f.a[i], bv, acc[i][j], f.idx[i], 0, 0);
            else
                acc[i][j] = __builtin_amdgcn_smfmac_i32_32x32x64_i8(f.a[i], bv, acc[i][j], f.idx[i], 0, 0);
        };

        Frags f0, f1;
        auto  stageBody = [&](uint32_t kt, uint32_t cur, uint32_t nxt) {
#pragma unroll
            for(uint32_t n = 0; n < 16; ++n)
            {
                mfmaAt(f0, n);
                readPiece(f1, cur, 1, n);
                __builtin_amdgcn_sched_barrier(0);
            }
            r355::waitVmcnt<LOADS_PER_STAGE>(); // stage kt + 1 has landed; the youngest 13 loads are stage kt + 2
            r355::ldsBarrier();
            const uint32_t refill = clampStage(kt + 3u);
#pragma unroll
            for(uint32_t n = 0; n < 16; ++n)
            {
                mfmaAt(f1, n);
                readPiece(f0, nxt, 0, n);
                if(n < LOADS_PER_STAGE)
                    issueLoad(refill, cur, n);
                __builtin_amdgcn_sched_barrier(0);
            }
        };

        constexpr uint32_t SLOT[3] = {0u, STAGE_BYTES, 2u * STAGE_BYTES};
#pragma unroll
        for(uint32_t st = 0; st < RING; ++st)
#pragma unroll
            for(uint32_t x = 0; x < LOADS_PER_STAGE; ++x)
                issueLoad(clampStage(st), SLOT[st], x);
        r355::waitVmcnt<2u * LOADS_PER_STAGE>();
        r355::ldsBarrier();
#pragma unroll
        for(uint32_t x = 0; x < 16; ++x)
            readPiece(f0, SLOT[0], 0, x);

        uint32_t kt = 0;
        for(uint32_t trips = numStages / 3u; trips > 0; --trips, kt += 3u)
        {
            stageBody(kt, SLOT[0], SLOT[1]);
            stageBody(kt + 1u, SLOT[1], SLOT[2]);
            stageBody(kt + 2u, SLOT[2], SLOT[0]);
        }
        const uint32_t rem = numStages - kt;
        if(rem > 0u)
        {
            stageBody(kt, SLOT[0], SLOT[1]);
            if(rem > 1u)
                stageBody(kt + 1u, SLOT[1], SLOT[2]);
        }
        // the clamped loads of the last stages are still landing in the slots the epilogue reuses
        r355::waitVmcnt<0>();
        r355::ldsBarrier();

        // ---- epilogue.  lane holds D(m = 8 (e / 4) + 4 g + e % 4, n = lane % 32) of each block:
        // four consecutive rows of one column.
        const AccE     alpha = static_cast<AccE>(p.alpha), beta = static_cast<AccE>(p.beta);
        const uint32_t m0 = tm * T_M + wm * 128u, n0 = tn * T_N + wn * 128u;
        using V4 = AccE __attribute__((ext_vector_type(4)));
        if(!p.dRow)
        {
            // col-major: a lane's four rows are contiguous
#pragma unroll
            for(uint32_t i = 0; i < 4; ++i)
#pragma unroll
                for(uint32_t j = 0; j < 4; ++j)
#pragma unroll
                    for(uint32_t q = 0; q < 4; ++q)
                    {
                        const uint32_t row = m0 + 32u * i + 8u * q + 4u * g, col = n0 + 32u * j + r32;
                        V4             out;
#pragma unroll
                        for(uint32_t e = 0; e < 4; ++e)
                            out[e] = alpha * acc[i][j][4 * q + e];
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
        // row-major: transpose through this wave's 26 KiB of the idle stage slots, 32 rows (one
        // block row i) at a time: rows of 128 x 4 bytes = 32 chunks, chunk c of row r in slot c ^ r.
        char* wl = lds + wave * 26624u;
#pragma unroll
        for(uint32_t i = 0; i < 4; ++i)
        {
#pragma unroll
            for(uint32_t j = 0; j < 4; ++j)
#pragma unroll
                for(uint32_t e = 0; e < 16; ++e)
                {
                    const uint32_t row = 8u * (e >> 2) + 4u * g + (e & 3u), col = 32u * j + r32;
                    *reinterpret_cast<AccE*>(wl + row * 512u + (((col >> 2) ^ row) * 16u) + (col & 3u) * 4u)
                        = alpha * acc[i][j][e];
                }
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for(uint32_t it = 0; it < 16; ++it)
            {
                const uint32_t L = it * 64u + lane, row = L >> 5, c = L & 31u;
                V4             v = *reinterpret_cast<const V4*>(wl + row * 512u + ((c ^ row) * 16u));
                const uint64_t off = (uint64_t)(m0 + 32u * i + row);
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

    bool tiledOk(const r355_gemm_args& g)
    {
        return g.kernel != R355_KERNEL_SIMPLE && (g.in_type == R355_I8 || g.in_type == R355_E4M3) && g.m % T_M == 0 && g.n % T_N == 0 && g.k % T_K == 0
               && g.layout_c == g.layout_d && (g.ldd % 4) == 0 && r355::aligned(g.d, 16)
               && (g.beta == 0.0 || ((g.ldc % 4) == 0 && r355::aligned(g.c, 16))) && r355::aligned(g.a_meta, 16);
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
        if(g.layout_a != R355_ROW_MAJOR || g.layout_b != R355_COL_MAJOR)
            return fail(R355_ERR_UNSUPPORTED, "sparse gemm: compressed A must be row-major and B col-major");
        if(!g.a_meta)
            return fail(R355_ERR_BAD_ARG, "sparse gemm: a_meta is null");
        const uint32_t es = w ? 2u : 1u, kStep = w ? 32u : 64u; // element bytes, dense k per matrix instruction
        if(g.m % 32 || g.n % 32 || g.k % kStep)
            return fail(R355_ERR_BAD_SIZE, "sparse gemm: m=%u n=%u must be multiples of 32 and k=%u of %u", g.m, g.n, g.k, kStep);
        if(!aligned(g.a, 16) || (g.lda * es) % 16 || !aligned(g.b, 16) || (g.ldb * es) % 16 || !aligned(g.a_meta, 4) || !aligned(g.d, 4))
            return fail(R355_ERR_MISALIGNED, "sparse gemm: values / B need 16-byte alignment, metadata 4-byte");
        if(g.kernel == R355_KERNEL_TILED_128)
            return fail(R355_ERR_UNSUPPORTED, "sparse gemm: there is no 128 x 128 sparse macro tile (R355_KERNEL_TILED is 256 x 256)");
        if(w && g.kernel == R355_KERNEL_TILED)
            return fail(R355_ERR_UNSUPPORTED, "sparse gemm (macro tile): 1-byte elements only");
        if(g.kernel == R355_KERNEL_TILED && !tiledOk(g))
            return fail(R355_ERR_BAD_SIZE, "sparse gemm (macro tile): m=%u n=%u must be multiples of 256, k=%u of 128, C/D same orientation and 16-byte aligned", g.m, g.n, g.k);
        if(plan && tiledOk(g))
        {
            plan->kernel       = R355_KERNEL_TILED;
            plan->macro_tile_m = T_M;
            plan->macro_tile_n = T_N;
            plan->macro_tile_k = T_K;
            plan->grid_x       = (((g.m / T_M) * (g.n / T_N) + 7u) / 8u) * 8u;
            plan->grid_y       = 1;
            plan->block_x      = T_THREADS;
            plan->block_y      = 1;
            plan->lds_bytes    = RING * STAGE_BYTES;
        }
        else if(plan)
        {
            plan->kernel       = R355_KERNEL_SIMPLE;
            plan->macro_tile_m = 32 * WAVES_X;
            plan->macro_tile_n = 32 * WAVES_Y;
            plan->macro_tile_k = (g.in_type == R355_F16 || g.in_type == R355_BF16) ? 32 : 64;
            plan->grid_x       = (g.m + 32 * WAVES_X - 1) / (32 * WAVES_X);
            plan->grid_y       = (g.n + 32 * WAVES_Y - 1) / (32 * WAVES_Y);
            plan->block_x      = WAVES_X * 64;
            plan->block_y      = WAVES_Y;
            plan->lds_bytes    = 0;
        }
        return R355_OK;
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
            p.lda = g.lda, p.ldb = g.ldb, p.ldc = g.ldc, p.ldd = g.ldd;
            p.alpha = g.alpha, p.beta = g.beta;
            p.tilesM = g.m / T_M, p.tilesN = g.n / T_N;
            p.dRow = g.layout_d == R355_ROW_MAJOR;
            const uint32_t grid = ((p.tilesM * p.tilesN + 7u) / 8u) * 8u;
            if(g.in_type == R355_E4M3)
                hipLaunchKernelGGL(sparseTiledKernel<true>, dim3(grid), dim3(T_THREADS), 0, stream, p);
            else
                hipLaunchKernelGGL(sparseTiledKernel<false>, dim3(grid), dim3(T_THREADS), 0, stream, p);
            return checkLaunch("sparse gemm (macro tile)");
        }
        dim3 block(WAVES_X * 64, WAVES_Y);
        dim3 grid((g.m + 32 * WAVES_X - 1) / (32 * WAVES_X), (g.n + 32 * WAVES_Y - 1) / (32 * WAVES_Y));
        auto* av = static_cast<const uint8_t*>(g.a);
        auto* am = static_cast<const uint8_t*>(g.a_meta);
        auto* bb = static_cast<const uint8_t*>(g.b);
        const bool cRow = g.layout_c == R355_ROW_MAJOR, dRow = g.layout_d == R355_ROW_MAJOR;
#define R355_SPARSE_LAUNCH(E)                                                                                       \
    hipLaunchKernelGGL(sparseBlockPerWave<SpElem::E>, grid, block, 0, stream, g.m, g.n, g.k, av, am, bb, g.c, g.d, g.lda, \
                       g.ldb, g.ldc, g.ldd, cRow, dRow, g.alpha, g.beta)
        switch(g.in_type)
        {
        case R355_E4M3: R355_SPARSE_LAUNCH(E4M3); break;
        case R355_F16: R355_SPARSE_LAUNCH(F16); break;
        case R355_BF16: R355_SPARSE_LAUNCH(BF16); break;
        default: R355_SPARSE_LAUNCH(I8); break;
        }
#undef R355_SPARSE_LAUNCH
        return checkLaunch("sparse gemm");
    }
} // namespace r355

namespace
{
    // An element counts as zero when all its bits are zero (a kept -0.0 stays a kept value: the round trip is exact).
    template <typename T>
    int compress24(const T* dense, uint32_t m, uint32_t k, T* values, uint8_t* meta)
    {
        if(!dense || !values || !meta)
            return r355::fail(R355_ERR_BAD_ARG, "compress_24: null pointer");
        if(k % 8u)
            return r355::fail(R355_ERR_BAD_SIZE, "compress_24: k=%u must be a multiple of 8", k);
        const uint32_t groups = k / 4u;
        for(uint32_t r = 0; r < m; ++r)
        {
            const T* src = dense + (size_t)r * k;
            T*       val = values + (size_t)r * (k / 2u);
            uint8_t* md  = meta + (size_t)r * (k / 8u);
            memset(md, 0, k / 8u);
            for(uint32_t g = 0; g < groups; ++g)
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
                val[2 * g]     = src[4 * g + pos[0]];
                val[2 * g + 1] = src[4 * g + pos[1]];
                md[g / 2] |= static_cast<uint8_t>((pos[0] | (pos[1] << 2)) << (4 * (g & 1u)));
            }
        }
        return R355_OK;
    }

    template <typename T>
    int decompress24(const T* values, const uint8_t* meta, uint32_t m, uint32_t k, T* dense)
    {
        if(!dense || !values || !meta)
            return r355::fail(R355_ERR_BAD_ARG, "decompress_24: null pointer");
        if(k % 8u)
            return r355::fail(R355_ERR_BAD_SIZE, "decompress_24: k=%u must be a multiple of 8", k);
        memset(dense, 0, (size_t)m * k * sizeof(T));
        for(uint32_t r = 0; r < m; ++r)
            for(uint32_t g = 0; g < k / 4u; ++g)
            {
                const uint32_t nib = (meta[(size_t)r * (k / 8u) + g / 2] >> (4 * (g & 1u))) & 0xFu;
                dense[(size_t)r * k + 4 * g + (nib & 3u)]  = values[(size_t)r * (k / 2u) + 2 * g];
                dense[(size_t)r * k + 4 * g + (nib >> 2)] = values[(size_t)r * (k / 2u) + 2 * g + 1];
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
