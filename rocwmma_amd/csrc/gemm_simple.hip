// Block-per-wave GEMM written against the fragment API: every wave owns one 16x16 or
// 32x32 block of D, streams A and B fragments straight from global memory, and applies
// alpha / beta element-wise on the accumulator fragment.  No LDS.
//
// Plays the role of samples/simple_hgemm.cpp:81-139 and
// test/gemm/gemm_PGR0_LB0_MP0_SB_NC/device/kernel_device_func.hpp:50-175 in the
// reference, for every supported type and all 16 layout combinations.  It is the
// correctness workhorse (latency-bound); the macro-tile kernels carry the throughput.
#include <rocwmma/rocwmma.hpp>

#include "common.hpp"

using namespace rocwmma;

namespace
{
    constexpr uint32_t WAVES_X = 2; // workgroup = (WAVES_X * 64, WAVES_Y) threads
    constexpr uint32_t WAVES_Y = 2;

    template <typename InT, typename OutT, typename CompT, typename LayoutA, typename LayoutB, uint32_t Blk, uint32_t BK>
    __global__ void __launch_bounds__(WAVES_X* WAVES_Y * 64) gemmBlockPerWave(uint32_t    m,
                                                                             uint32_t    n,
                                                                             uint32_t    k,
                                                                             InT const*  a,
                                                                             InT const*  b,
                                                                             OutT const* c,
                                                                             OutT*       d,
                                                                             uint32_t    lda,
                                                                             uint32_t    ldb,
                                                                             uint32_t    ldc,
                                                                             uint32_t    ldd,
                                                                             layout_t    layoutC,
                                                                             layout_t    layoutD,
                                                                             CompT       alpha,
                                                                             CompT       beta)
    {
        using FragA   = fragment<matrix_a, Blk, Blk, BK, InT, LayoutA>;
        using FragB   = fragment<matrix_b, Blk, Blk, BK, InT, LayoutB>;
        using FragAcc = fragment<accumulator, Blk, Blk, BK, CompT>;
        using FragC   = fragment<accumulator, Blk, Blk, BK, OutT>;
        using MapA    = GetDataLayout_t<FragA>;
        using MapB    = GetDataLayout_t<FragB>;

        const uint32_t row = (blockIdx.x * WAVES_X + threadIdx.x / Constants::AMDGCN_WAVE_SIZE) * Blk;
        const uint32_t col = (blockIdx.y * WAVES_Y + threadIdx.y) * Blk;
        if(row >= m || col >= n)
            return;

        FragA   fragA;
        FragB   fragB;
        FragAcc fragAcc;
        fill_fragment(fragAcc, static_cast<CompT>(0));

        // 64-bit offsets: rows * ld of an operand that fits 288 GB of HBM can exceed 2^32 elements (the
        // fragment API's own fromMatrixCoord is 32-bit like the reference's)
        constexpr bool aRow  = std::is_same_v<LayoutA, row_major>;
        constexpr bool bRow  = std::is_same_v<LayoutB, row_major>;
        const InT*     pa    = a + (aRow ? (uint64_t)row * lda : (uint64_t)row);
        const InT*     pb    = b + (bRow ? (uint64_t)col : (uint64_t)col * ldb);
        const uint64_t stepA = aRow ? (uint64_t)BK : (uint64_t)BK * lda;
        const uint64_t stepB = bRow ? (uint64_t)BK * ldb : (uint64_t)BK;

        for(uint32_t i = 0; i < k; i += BK)
        {
            load_matrix_sync(fragA, pa, lda);
            load_matrix_sync(fragB, pb, ldb);
            mma_sync(fragAcc, fragA, fragB, fragAcc);
            pa += stepA;
            pb += stepB;
        }

        const uint64_t offC = layoutC == mem_row_major ? (uint64_t)row * ldc + col : (uint64_t)col * ldc + row;
        const uint64_t offD = layoutD == mem_row_major ? (uint64_t)row * ldd + col : (uint64_t)col * ldd + row;

        FragC fragC;
        if(beta != static_cast<CompT>(0))
        {
            load_matrix_sync(fragC, c + offC, ldc, layoutC);
#pragma unroll
            for(uint32_t i = 0; i < FragC::num_elements; ++i)
                fragC.x[i] = convert<OutT>(
                    static_cast<CompT>(alpha * fragAcc.x[i] + beta * convert<CompT>(fragC.x[i])));
        }
        else
        {
#pragma unroll
            for(uint32_t i = 0; i < FragC::num_elements; ++i)
                fragC.x[i] = convert<OutT>(static_cast<CompT>(alpha * fragAcc.x[i]));
        }
        store_matrix_sync(d + offD, fragC, ldd, layoutD);
    }

    // Smallest K extent of one MFMA for a block size (the kernel's K granularity)
    template <typename InT, uint32_t Blk>
    constexpr uint32_t blockK()
    {
        if constexpr(sizeof(InT) == 2)
            return Blk == 32 ? 16 : 16;
        else if constexpr(std::is_same_v<InT, int8_t>)
            return Blk == 32 ? 32 : 32;
        else if constexpr(sizeof(InT) == 1)
            return Blk == 32 ? 16 : 32;
        else
            return Blk == 32 ? 2 : 4; // f32; f64 exists for 16 x 16 blocks only (K 4)
    }

    template <typename InT, typename OutT, typename CompT, typename LayoutA, typename LayoutB, uint32_t Blk>
    int launchTyped(const r355_gemm_args& g, hipStream_t stream)
    {
        constexpr uint32_t BK = blockK<InT, Blk>();
        dim3               block(WAVES_X * 64, WAVES_Y);
        dim3               grid(ceilDiv(g.m, Blk * WAVES_X), ceilDiv(g.n, Blk * WAVES_Y));
        hipLaunchKernelGGL((gemmBlockPerWave<InT, OutT, CompT, LayoutA, LayoutB, Blk, BK>),
                           grid,
                           block,
                           0,
                           stream,
                           g.m,
                           g.n,
                           g.k,
                           static_cast<const InT*>(g.a),
                           static_cast<const InT*>(g.b),
                           static_cast<const OutT*>(g.c),
                           static_cast<OutT*>(g.d),
                           g.lda,
                           g.ldb,
                           g.ldc,
                           g.ldd,
                           g.layout_c == R355_ROW_MAJOR ? mem_row_major : mem_col_major,
                           g.layout_d == R355_ROW_MAJOR ? mem_row_major : mem_col_major,
                           static_cast<CompT>(g.alpha),
                           static_cast<CompT>(g.beta));
        return r355::checkLaunch("gemm (block per wave)");
    }

    template <typename InT, typename OutT, typename CompT, uint32_t Blk>
    int launchLayouts(const r355_gemm_args& g, hipStream_t stream)
    {
        const bool aRow = g.layout_a == R355_ROW_MAJOR, bRow = g.layout_b == R355_ROW_MAJOR;
        if(aRow && bRow)
            return launchTyped<InT, OutT, CompT, row_major, row_major, Blk>(g, stream);
        if(aRow && !bRow)
            return launchTyped<InT, OutT, CompT, row_major, col_major, Blk>(g, stream);
        if(!aRow && bRow)
            return launchTyped<InT, OutT, CompT, col_major, row_major, Blk>(g, stream);
        return launchTyped<InT, OutT, CompT, col_major, col_major, Blk>(g, stream);
    }

    template <typename InT, typename OutT, typename CompT>
    int launchBlocks(const r355_gemm_args& g, hipStream_t stream, uint32_t blk)
    {
        if constexpr(std::is_same_v<InT, float64_t>)
            return launchLayouts<InT, OutT, CompT, 16>(g, stream);
        else
            return blk == 32 ? launchLayouts<InT, OutT, CompT, 32>(g, stream)
                             : launchLayouts<InT, OutT, CompT, 16>(g, stream);
    }

    uint32_t kGranule(int32_t inType, uint32_t blk)
    {
        switch(inType)
        {
        case R355_F16:
        case R355_BF16: return 16;
        case R355_I8: return 32;
        case R355_E4M3:
        case R355_E5M2: return blk == 32 ? 16 : 32;
        case R355_F32: return blk == 32 ? 2 : 4;
        case R355_F64: return 4;
        default: return 0;
        }
    }

    // Widest vector a fragment access may use: pointers and leading dimensions must keep it aligned
    uint32_t vectorBytes(int32_t inType)
    {
        return inType == R355_F32 ? 4 : (inType == R355_F64 ? 8 : 16);
    }

    uint32_t pickBlock(const r355_gemm_args& g)
    {
        if(g.in_type != R355_F64 && g.m % 32 == 0 && g.n % 32 == 0 && g.k % kGranule(g.in_type, 32) == 0)
            return 32;
        if(g.m % 16 == 0 && g.n % 16 == 0 && g.k % kGranule(g.in_type, 16) == 0)
            return 16;
        return 0;
    }

    bool typePairOk(int32_t in, int32_t out)
    {
        switch(in)
        {
        case R355_F16: return out == R355_F32 || out == R355_F16;
        case R355_BF16: return out == R355_F32 || out == R355_BF16;
        case R355_E4M3:
        case R355_E5M2: return out == R355_F32;
        case R355_I8: return out == R355_I32 || out == R355_I8;
        case R355_F32: return out == R355_F32;
        case R355_F64: return out == R355_F64;
        default: return false;
        }
    }
} // namespace

namespace r355
{
    int gemmSimpleCheck(const r355_gemm_args& g, r355_gemm_plan* plan)
    {
        if(!typePairOk(g.in_type, g.out_type))
            return fail(R355_ERR_UNSUPPORTED, "gemm: no kernel for in_type %d -> out_type %d", g.in_type, g.out_type);
        const uint32_t blk = pickBlock(g);
        if(blk == 0)
            return fail(R355_ERR_BAD_SIZE,
                        "gemm: m=%u n=%u must be multiples of 16 and k=%u a multiple of %u",
                        g.m, g.n, g.k, kGranule(g.in_type, 16));
        // Fragment loads move up to 16 bytes along the contiguous dimension
        const uint32_t eb = dtypeBytes(g.in_type), ob = dtypeBytes(g.out_type);
        const uint32_t va = g.layout_a == R355_ROW_MAJOR ? vectorBytes(g.in_type) : eb;
        const uint32_t vb = g.layout_b == R355_COL_MAJOR ? vectorBytes(g.in_type) : eb;
        // accumulator fragments hold 4 consecutive rows per lane (f64: one row per register)
        const uint32_t accRun = g.out_type == R355_F64 ? 1u : 4u;
        const uint32_t vd = g.layout_d == R355_COL_MAJOR ? accRun * ob : ob;
        const uint32_t vc = g.layout_c == R355_COL_MAJOR ? accRun * ob : ob;
        if(!aligned(g.a, va) || (g.lda * eb) % va || !aligned(g.b, vb) || (g.ldb * eb) % vb
           || !aligned(g.d, vd) || (g.ldd * ob) % vd
           || (g.beta != 0.0 && (!aligned(g.c, vc) || (g.ldc * ob) % vc)))
            return fail(R355_ERR_MISALIGNED, "gemm: pointers / leading dimensions must keep %u-byte vectors aligned", va > vb ? va : vb);
        if(plan)
        {
            plan->kernel       = R355_KERNEL_SIMPLE;
            plan->macro_tile_m = blk * WAVES_X;
            plan->macro_tile_n = blk * WAVES_Y;
            plan->macro_tile_k = kGranule(g.in_type, blk);
            plan->grid_x       = (g.m + blk * WAVES_X - 1) / (blk * WAVES_X);
            plan->grid_y       = (g.n + blk * WAVES_Y - 1) / (blk * WAVES_Y);
            plan->block_x      = WAVES_X * 64;
            plan->block_y      = WAVES_Y;
            plan->lds_bytes    = 0;
        }
        return R355_OK;
    }

    int gemmSimpleLaunch(const r355_gemm_args& g, hipStream_t stream)
    {
        const uint32_t blk = pickBlock(g);
        switch(g.in_type)
        {
        case R355_F16:
            return g.out_type == R355_F32 ? launchBlocks<float16_t, float32_t, float32_t>(g, stream, blk)
                                          : launchBlocks<float16_t, float16_t, float32_t>(g, stream, blk);
        case R355_BF16:
            return g.out_type == R355_F32 ? launchBlocks<bfloat16_t, float32_t, float32_t>(g, stream, blk)
                                          : launchBlocks<bfloat16_t, bfloat16_t, float32_t>(g, stream, blk);
        case R355_E4M3: return launchBlocks<float8_t, float32_t, float32_t>(g, stream, blk);
        case R355_E5M2: return launchBlocks<bfloat8_t, float32_t, float32_t>(g, stream, blk);
        case R355_I8:
            return g.out_type == R355_I32 ? launchBlocks<int8_t, int32_t, int32_t>(g, stream, blk)
                                          : launchBlocks<int8_t, int8_t, int32_t>(g, stream, blk);
        case R355_F32: return launchBlocks<float32_t, float32_t, float32_t>(g, stream, blk);
        case R355_F64: return launchBlocks<float64_t, float64_t, float64_t>(g, stream, blk);
        default: return fail(R355_ERR_UNSUPPORTED, "gemm: unknown in_type %d", g.in_type);
        }
    }
} // namespace r355
