// 2:4 structured-sparse GEMM on gfx950 sparse matrix cores (v_smfmac_*), plus the host-side
// compressor.  The reference has no sparse path; the storage format is defined here.
//
// A (m x k, row-major, 1-byte elements) keeps 2 of every aligned group of 4 along k:
//   values  m x k/2   the kept pair of each group, in position order
//   meta    m x k/8   one nibble per group = idx0 | idx1 << 2 (idx0 < idx1), even group in the
//                     low nibble -- 32 bits cover 32 dense k, which is exactly the index
//                     register one lane feeds to v_smfmac_*_32x32x64 for its 16 kept values.
// B is dense, col-major (k contiguous); D row- or col-major.
//
// Kernel: one 32 x 32 block of D per wave, operands streamed from global memory
// (lane = row / column, 16 kept bytes + 4 index bytes of A and 2 x 16 dense bytes of B per
// 64-wide K step).  Operand formats of v_smfmac_*_32x32x64 as measured on MI355X: index
// bits [2 p + 1 : 2 p] give the position within its group of 4 of kept byte p of the lane.
#include <hip/hip_runtime.h>

#include <cstring>

#include "common.hpp"

namespace
{
    using i32x4  = int __attribute__((ext_vector_type(4)));
    using i32x8  = int __attribute__((ext_vector_type(8)));
    using i32x16 = int __attribute__((ext_vector_type(16)));
    using f32x16 = float __attribute__((ext_vector_type(16)));

    constexpr uint32_t WAVES_X = 2, WAVES_Y = 2;

    template <bool FP8>
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
                                                                               float          alphaF,
                                                                               float          betaF)
    {
        using Acc  = std::conditional_t<FP8, f32x16, i32x16>;
        using AccE = std::conditional_t<FP8, float, int>;
        const uint32_t lane = threadIdx.x & 63u;
        const uint32_t row0 = (blockIdx.x * WAVES_X + threadIdx.x / 64u) * 32u;
        const uint32_t col0 = (blockIdx.y * WAVES_Y + threadIdx.y) * 32u;
        if(row0 >= m || col0 >= n)
            return;
        const uint32_t idx = lane & 31u, g = lane >> 5;

        const uint8_t* pa = aVals + (uint64_t)(row0 + idx) * lda + 16u * g;
        const uint8_t* pm = aMeta + (uint64_t)(row0 + idx) * (k / 8u) + 4u * g;
        // The instruction pairs A's lane group g, kept bytes [8 q, 8 q + 8) with B's lane group q,
        // dense bytes [16 g, 16 g + 16).  With A's lane group g holding the kept values of dense
        // k in [32 g, 32 g + 32), B's lane group h therefore holds dense k in [16 h, 16 h + 16)
        // and [32 + 16 h, 48 + 16 h) of each 64-wide step.
        const uint8_t* pb = b + (uint64_t)(col0 + idx) * ldb + 16u * g;

        Acc acc;
#pragma unroll
        for(uint32_t e = 0; e < 16; ++e)
            acc[e] = 0;

        for(uint32_t kd = 0; kd < k; kd += 64u)
        {
            const i32x4 av   = *reinterpret_cast<const i32x4*>(pa + kd / 2u);
            const int   meta = *reinterpret_cast<const int*>(pm + kd / 8u);
            const i32x4 b0   = *reinterpret_cast<const i32x4*>(pb + kd);
            const i32x4 b1   = *reinterpret_cast<const i32x4*>(pb + kd + 32u);
            const i32x8 bv   = {b0[0], b0[1], b0[2], b0[3], b1[0], b1[1], b1[2], b1[3]};
            if constexpr(FP8)
                acc = __builtin_amdgcn_smfmac_f32_32x32x64_fp8_fp8(av, bv, acc, meta, 0, 0);
            else
                acc = __builtin_amdgcn_smfmac_i32_32x32x64_i8(av, bv, acc, meta, 0, 0);
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
} // namespace

namespace r355
{
    int gemmSparseCheck(const r355_gemm_args& g, r355_gemm_plan* plan)
    {
        const bool i8 = g.in_type == R355_I8 && g.out_type == R355_I32;
        const bool f8 = g.in_type == R355_E4M3 && g.out_type == R355_F32;
        if(!i8 && !f8)
            return fail(R355_ERR_UNSUPPORTED, "sparse gemm: supported types are i8 -> i32 and e4m3 -> f32");
        if(g.layout_a != R355_ROW_MAJOR || g.layout_b != R355_COL_MAJOR)
            return fail(R355_ERR_UNSUPPORTED, "sparse gemm: compressed A must be row-major and B col-major");
        if(!g.a_meta)
            return fail(R355_ERR_BAD_ARG, "sparse gemm: a_meta is null");
        if(g.m % 32 || g.n % 32 || g.k % 64)
            return fail(R355_ERR_BAD_SIZE, "sparse gemm: m=%u n=%u must be multiples of 32 and k=%u of 64", g.m, g.n, g.k);
        if(!aligned(g.a, 16) || g.lda % 16 || !aligned(g.b, 16) || g.ldb % 16 || !aligned(g.a_meta, 4) || !aligned(g.d, 4))
            return fail(R355_ERR_MISALIGNED, "sparse gemm: values / B need 16-byte alignment, metadata 4-byte");
        if(plan)
        {
            plan->kernel       = R355_KERNEL_SIMPLE;
            plan->macro_tile_m = 32 * WAVES_X;
            plan->macro_tile_n = 32 * WAVES_Y;
            plan->macro_tile_k = 64;
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
        dim3 block(WAVES_X * 64, WAVES_Y);
        dim3 grid((g.m + 32 * WAVES_X - 1) / (32 * WAVES_X), (g.n + 32 * WAVES_Y - 1) / (32 * WAVES_Y));
        auto* av = static_cast<const uint8_t*>(g.a);
        auto* am = static_cast<const uint8_t*>(g.a_meta);
        auto* bb = static_cast<const uint8_t*>(g.b);
        const bool cRow = g.layout_c == R355_ROW_MAJOR, dRow = g.layout_d == R355_ROW_MAJOR;
        if(g.in_type == R355_E4M3)
            hipLaunchKernelGGL(sparseBlockPerWave<true>, grid, block, 0, stream, g.m, g.n, g.k, av, am, bb, g.c, g.d,
                               g.lda, g.ldb, g.ldc, g.ldd, cRow, dRow, g.alpha, g.beta);
        else
            hipLaunchKernelGGL(sparseBlockPerWave<false>, grid, block, 0, stream, g.m, g.n, g.k, av, am, bb, g.c, g.d,
                               g.lda, g.ldb, g.ldc, g.ldd, cRow, dRow, g.alpha, g.beta);
        return checkLaunch("sparse gemm");
    }
} // namespace r355

extern "C" int r355_compress_24(const uint8_t* dense, uint32_t m, uint32_t k, uint8_t* values, uint8_t* meta)
{
    if(!dense || !values || !meta)
        return r355::fail(R355_ERR_BAD_ARG, "compress_24: null pointer");
    if(k % 8u)
        return r355::fail(R355_ERR_BAD_SIZE, "compress_24: k=%u must be a multiple of 8", k);
    const uint32_t groups = k / 4u;
    for(uint32_t r = 0; r < m; ++r)
    {
        const uint8_t* src = dense + (size_t)r * k;
        uint8_t*       val = values + (size_t)r * (k / 2u);
        uint8_t*       md  = meta + (size_t)r * (k / 8u);
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

extern "C" int r355_decompress_24(const uint8_t* values, const uint8_t* meta, uint32_t m, uint32_t k, uint8_t* dense)
{
    if(!dense || !values || !meta)
        return r355::fail(R355_ERR_BAD_ARG, "decompress_24: null pointer");
    if(k % 8u)
        return r355::fail(R355_ERR_BAD_SIZE, "decompress_24: k=%u must be a multiple of 8", k);
    memset(dense, 0, (size_t)m * k);
    for(uint32_t r = 0; r < m; ++r)
        for(uint32_t g = 0; g < k / 4u; ++g)
        {
            const uint32_t nib = (meta[(size_t)r * (k / 8u) + g / 2] >> (4 * (g & 1u))) & 0xFu;
            dense[(size_t)r * k + 4 * g + (nib & 3u)]  = values[(size_t)r * (k / 2u) + 2 * g];
            dense[(size_t)r * k + 4 * g + (nib >> 2)] = values[(size_t)r * (k / 2u) + 2 * g + 1];
        }
    return R355_OK;
}
