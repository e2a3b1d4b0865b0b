// DLRM dot-interaction forward and backward for gfx950.
//
// Forward takes the place of test/dlrm/device/dlrm_dot_fwd.hpp:35-138 (and the LDS variant
// dlrm_dot_fwd_lds.hpp:35-190, samples/simple_dlrm.cpp:184-284).  The reference gives each
// wave one 16x16 tile of X X^T, stores f32 tiles to a global scratch `acc[b][m][m]` and
// re-reads them to scatter the lower triangle.  This path is HBM-bound (about 24 flop per
// byte), so the kernel is organised around memory traffic instead:
//
//   * one wave owns one sample at a time; a workgroup (4 waves) owns 8 consecutive samples,
//     whose outputs form one contiguous, 16-byte aligned run of 8 * (k + m(m-1)/2) elements;
//   * X (m x k, m <= 32) is read once with fully coalesced 128-bit loads (both samples of a
//     wave are requested before either is consumed), parked in LDS with a per-row XOR swizzle,
//     and fed to v_mfma_f32_32x32x16 with the same register as both operands (X X^T): k / 16
//     matrix instructions, one 128-bit LDS read each; lanes of rows >= m feed zeros, which is
//     the 27 -> 32 padding;
//   * the strict lower triangle and the copied first row are assembled in an LDS image of
//     the output and leave with coalesced 128-bit stores.  No global scratch.
//
// Backward takes the place of test/dlrm/device/dlrm_dot_bwd.hpp:35-176: the upstream
// triangle is rebuilt symmetric in LDS (trilReconstruct) and multiplied into X with the
// same matrix instruction, again without global scratch.
#include <hip/hip_runtime.h>

#include "common.hpp"

namespace
{
    using f32x16 = float __attribute__((ext_vector_type(16)));
    using i32x4  = int __attribute__((ext_vector_type(4)));
    using f16x8  = _Float16 __attribute__((ext_vector_type(8)));
    using bf16x8 = __bf16 __attribute__((ext_vector_type(8)));

    constexpr uint32_t WAVES          = 4;
    constexpr uint32_t THREADS        = WAVES * 64;
    constexpr uint32_t SAMPLES_PER_WG = 8; // 8 * out_row_bytes is a multiple of 16 for every (m, k)
    constexpr uint32_t MAX_M          = 32;
    constexpr uint32_t MAX_K          = 256;

    template <bool BF16>
    __device__ inline f32x16 mfma16(f32x16 acc, i32x4 x, i32x4 y)
    {
        if constexpr(BF16)
            return __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                __builtin_bit_cast(bf16x8, x), __builtin_bit_cast(bf16x8, y), acc, 0, 0, 0);
        else
            return __builtin_amdgcn_mfma_f32_32x32x16_f16(
                __builtin_bit_cast(f16x8, x), __builtin_bit_cast(f16x8, y), acc, 0, 0, 0);
    }

    template <bool BF16>
    __device__ inline uint16_t roundOut(float v)
    {
        if constexpr(BF16)
            return __builtin_bit_cast(uint16_t, static_cast<__bf16>(v));
        else
            return __builtin_bit_cast(uint16_t, static_cast<_Float16>(v));
    }

    // K is a template parameter (32, 64, 128, 256): rows of X are K * 2 bytes = K / 8 chunks.
    // ROWS (28 or 32) bounds m: the LDS image of a sample holds ROWS rows, which at m <= 28 and
    // K = 128 lets four workgroups share a CU instead of three.
    template <bool BF16, uint32_t K, uint32_t ROWS>
    __global__ void __launch_bounds__(THREADS)
        dlrmFwdKernel(const uint16_t* __restrict__ in, uint16_t* __restrict__ out, uint32_t m, uint32_t batch)
    {
        constexpr uint32_t ROW_CHUNKS = K / 8; // 16-byte chunks per row
        constexpr uint32_t X_BYTES    = ROWS * K * 2; // LDS image of one sample
        constexpr uint32_t MAX_OUT    = K + ROWS * (ROWS - 1) / 2;

        __shared__ __attribute__((aligned(16))) char     xLds[WAVES][X_BYTES];
        __shared__ __attribute__((aligned(16))) uint16_t outLds[SAMPLES_PER_WG * MAX_OUT + 8];

        const uint32_t tid       = threadIdx.x;
        const uint32_t lane      = tid & 63u;
        const uint32_t wave      = tid >> 6;
        const uint32_t outStride = K + m * (m - 1) / 2; // elements per sample
        const uint32_t b0        = blockIdx.x * SAMPLES_PER_WG;
        const uint32_t inChunks  = m * ROW_CHUNKS; // 16-byte chunks of one sample

        char* xw = xLds[wave];
        // rows m..31 of the 32 x 32 product are padding: their lanes feed zeros (see below)

        // Both samples of this wave are requested from HBM before either is consumed: the kernel is
        // bandwidth-bound, and bytes in flight per CU are what keeps HBM busy.
        constexpr uint32_t PER_WAVE   = SAMPLES_PER_WG / WAVES; // 2
        constexpr uint32_t MAX_CHUNKS = (ROWS * ROW_CHUNKS + 63u) / 64u; // loads per lane per sample
        i32x4              stash[PER_WAVE][MAX_CHUNKS];
#pragma unroll
        for(uint32_t q = 0; q < PER_WAVE; ++q)
        {
            const uint32_t b = b0 + wave + q * WAVES;
            if(b < batch)
            {
                const char* src = reinterpret_cast<const char*>(in) + (uint64_t)b * m * K * 2u;
#pragma unroll
                for(uint32_t j = 0; j < MAX_CHUNKS; ++j)
                {
                    const uint32_t c = j * 64u + lane;
                    if(c < inChunks)
                        stash[q][j] = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(src + c * 16u)); // read once
                }
            }
        }

#pragma unroll
        for(uint32_t q = 0; q < PER_WAVE; ++q)
        {
            const uint32_t sIdx = wave + q * WAVES;
            const uint32_t b    = b0 + sIdx;
            if(b >= batch)
                break;
            // ---- X -> LDS: chunk c of the sample goes to row c / ROW_CHUNKS, slot (c % ROW_CHUNKS) ^ (row % 16)
#pragma unroll
            for(uint32_t j = 0; j < MAX_CHUNKS; ++j)
            {
                const uint32_t c = j * 64u + lane;
                if(c < inChunks)
                {
                    const uint32_t row  = c / ROW_CHUNKS, col = c % ROW_CHUNKS;
                    const uint32_t slot = col ^ (row & (ROW_CHUNKS - 1u) & 15u);
                    *reinterpret_cast<i32x4*>(xw + (row * ROW_CHUNKS + slot) * 16u) = stash[q][j];
                }
            }
            __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0): this wave's LDS writes are done
            __builtin_amdgcn_wave_barrier();

            // ---- Gram matrix: acc(i, j) = sum_k X(i, k) X(j, k)
            f32x16         acc   = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            const bool     valid = (lane & 31u) < m;
            const uint32_t row   = valid ? (lane & 31u) : 0u; // padding lanes read row 0 and discard it
#pragma unroll
            for(uint32_t s = 0; s < K / 16; ++s)
            {
                const uint32_t col  = 2u * s + (lane >> 5);
                const uint32_t slot = col ^ (row & (ROW_CHUNKS - 1u) & 15u);
                i32x4          x    = *reinterpret_cast<const i32x4*>(xw + (row * ROW_CHUNKS + slot) * 16u);
                if(!valid)
                    x = i32x4{0, 0, 0, 0};
                acc = mfma16<BF16>(acc, x, x);
            }

            // ---- output image: first row, then strict lower triangle (i, j < i) row-major
            uint16_t* o = outLds + sIdx * outStride;
            for(uint32_t e = lane; e < K; e += 64)
                o[e] = reinterpret_cast<const uint16_t*>(xw)[e]; // row 0 is stored unswizzled
            const uint32_t j = lane & 31u;
#pragma unroll
            for(uint32_t r = 0; r < 16; ++r)
            {
                const uint32_t i = 8u * (r >> 2) + 4u * (lane >> 5) + (r & 3u);
                if(j < i && i < m)
                    o[K + i * (i - 1u) / 2u + j] = roundOut<BF16>(acc[r]);
            }
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __builtin_amdgcn_wave_barrier();
        }
        __syncthreads();

        // ---- coalesced copy-out of the workgroup's samples
        const uint32_t nSamples = (batch - b0) < SAMPLES_PER_WG ? (batch - b0) : SAMPLES_PER_WG;
        const uint32_t total    = nSamples * outStride; // elements
        uint16_t*      dst      = out + (uint64_t)b0 * outStride;
        const uint32_t vecs     = total / 8u;
        for(uint32_t v = tid; v < vecs; v += THREADS)
            __builtin_nontemporal_store(reinterpret_cast<const i32x4*>(outLds)[v], reinterpret_cast<i32x4*>(dst) + v);
        for(uint32_t e = vecs * 8u + tid; e < total; e += THREADS)
            dst[e] = outLds[e];
    }

    // f32 variant: one sample per wave, four per workgroup (4 * out_row_bytes is a multiple of 16),
    // v_mfma_f32_32x32x2f32 on an LDS image of X with 16-byte chunks XOR-swizzled by row.
    template <uint32_t K>
    __global__ void __launch_bounds__(THREADS)
        dlrmFwdF32Kernel(const float* __restrict__ in, float* __restrict__ out, uint32_t m, uint32_t batch)
    {
        constexpr uint32_t ROW_CHUNKS = K / 4; // 16-byte chunks per row
        constexpr uint32_t MAX_OUT    = K + MAX_M * (MAX_M - 1) / 2;
        constexpr uint32_t MAX_CHUNKS = (MAX_M * ROW_CHUNKS + 63u) / 64u;
        using f32x4                   = float __attribute__((ext_vector_type(4)));

        __shared__ __attribute__((aligned(16))) float xLds[WAVES][MAX_M * K];
        __shared__ __attribute__((aligned(16))) float outLds[WAVES * MAX_OUT + 4];

        const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
        const uint32_t outStride = K + m * (m - 1) / 2;
        const uint32_t b0        = blockIdx.x * WAVES;
        const uint32_t inChunks  = m * ROW_CHUNKS;
        const uint32_t b         = b0 + wave;
        char*          xw        = reinterpret_cast<char*>(xLds[wave]);

        if(b < batch)
        {
            const char* src = reinterpret_cast<const char*>(in) + (uint64_t)b * m * K * 4u;
            f32x4       stash[MAX_CHUNKS];
#pragma unroll
            for(uint32_t j = 0; j < MAX_CHUNKS; ++j)
            {
                const uint32_t c = j * 64u + lane;
                if(c < inChunks)
                    stash[j] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(src + c * 16u));
            }
#pragma unroll
            for(uint32_t j = 0; j < MAX_CHUNKS; ++j)
            {
                const uint32_t c = j * 64u + lane;
                if(c < inChunks)
                {
                    const uint32_t row = c / ROW_CHUNKS, col = c % ROW_CHUNKS;
                    *reinterpret_cast<f32x4*>(xw + (row * ROW_CHUNKS + (col ^ (row & (ROW_CHUNKS - 1u) & 31u))) * 16u) = stash[j];
                }
            }
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __builtin_amdgcn_wave_barrier();

            f32x16         acc   = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            const bool     valid = (lane & 31u) < m;
            const uint32_t row   = valid ? (lane & 31u) : 0u;
#pragma unroll 8
            for(uint32_t s = 0; s < K / 2; ++s)
            {
                const uint32_t kk  = 2u * s + (lane >> 5);
                const uint32_t col = kk >> 2;
                float          x   = *reinterpret_cast<const float*>(
                    xw + (row * ROW_CHUNKS + (col ^ (row & (ROW_CHUNKS - 1u) & 31u))) * 16u + (kk & 3u) * 4u);
                if(!valid)
                    x = 0.0f;
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(x, x, acc, 0, 0, 0);
            }

            float* o = outLds + wave * outStride;
            for(uint32_t e = lane; e < K; e += 64)
                o[e] = reinterpret_cast<const float*>(xw)[e]; // row 0 is stored unswizzled
            const uint32_t j = lane & 31u;
#pragma unroll
            for(uint32_t r = 0; r < 16; ++r)
            {
                const uint32_t i = 8u * (r >> 2) + 4u * (lane >> 5) + (r & 3u);
                if(j < i && i < m)
                    o[K + i * (i - 1u) / 2u + j] = acc[r];
            }
        }
        __syncthreads();
        const uint32_t nSamples = (batch - b0) < WAVES ? (batch - b0) : WAVES;
        const uint32_t total    = nSamples * outStride;
        float*         dst      = out + (uint64_t)b0 * outStride;
        const uint32_t vecs     = total / 4u;
        for(uint32_t v = tid; v < vecs; v += THREADS)
            __builtin_nontemporal_store(reinterpret_cast<const f32x4*>(outLds)[v], reinterpret_cast<f32x4*>(dst) + v);
        for(uint32_t e = vecs * 4u + tid; e < total; e += THREADS)
            dst[e] = outLds[e];
    }

    // Backward: S = T + T^T (T = strict lower triangle from the upstream gradient),
    // grad(m x k) = S X, computed as acc(i, c) = sum_j S(i, j) X(j, c) per 32-column slab of k.
    template <bool BF16, uint32_t K>
    __global__ void __launch_bounds__(THREADS) dlrmBwdKernel(const uint16_t* __restrict__ in,
                                                            const uint16_t* __restrict__ upstream,
                                                            uint16_t* __restrict__ mlpGrad,
                                                            uint16_t* __restrict__ inGrad,
                                                            uint32_t m,
                                                            uint32_t batch)
    {
        // S: 32 x 32 elements, row i holds S(i, 0..31) -> K-contiguous operand X-role "A" (32 x 32, K = j)
        // X^T is needed as the other operand: lane (c = lane % 32, j-run) -> X(j, c) for 8 consecutive j;
        // X is stored (j, c) row-major in memory, i.e. contiguous along c: keep X in LDS as [j][c]
        // and gather the 8 values of a lane's j-run with 16-bit LDS reads.
        __shared__ uint16_t sLds[WAVES][32 * 32];
        __shared__ uint16_t xLds[WAVES][32 * MAX_K];

        const uint32_t tid      = threadIdx.x;
        const uint32_t lane     = tid & 63u;
        const uint32_t wave     = tid >> 6;
        const uint32_t upStride = K + m * (m - 1) / 2;
        uint16_t*      sw       = sLds[wave];
        uint16_t*      xw       = xLds[wave];

        for(uint32_t b = blockIdx.x * WAVES + wave; b < batch; b += gridDim.x * WAVES)
        {
            const uint16_t* up = upstream + (uint64_t)b * upStride;
            const uint16_t* x  = in + (uint64_t)b * m * K;
            for(uint32_t e = lane; e < K; e += 64)
                mlpGrad[(uint64_t)b * K + e] = up[e];
            // symmetric S with zero diagonal and zero padding
            for(uint32_t e = lane; e < 32 * 32; e += 64)
            {
                const uint32_t i = e >> 5, j = e & 31u;
                uint16_t       v = 0;
                if(i < m && j < m && i != j)
                {
                    const uint32_t hi = i > j ? i : j, lo = i > j ? j : i;
                    v                 = up[K + hi * (hi - 1u) / 2u + lo];
                }
                sw[e] = v;
            }
            for(uint32_t e = lane; e < 32 * K; e += 64)
                xw[e] = e < m * K ? x[e] : (uint16_t)0;
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __builtin_amdgcn_wave_barrier();

            const uint32_t idx = lane & 31u, run = 8u * (lane >> 5);
            for(uint32_t c0 = 0; c0 < K; c0 += 32)
            {
                f32x16 acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
                for(uint32_t s = 0; s < 2; ++s) // j = 16 s + run .. + 7
                {
                    // swapped operands: "rows" of the instruction = c, "cols" = i, so that a lane
                    // ends up with 4 consecutive c of one output row i
                    union
                    {
                        uint16_t h[8];
                        i32x4    v;
                    } xo, so;
#pragma unroll
                    for(uint32_t e = 0; e < 8; ++e)
                    {
                        const uint32_t j = 16u * s + run + e;
                        xo.h[e]          = xw[j * K + c0 + idx]; // X(j, c0 + idx)
                        so.h[e]          = sw[idx * 32u + j]; // S(idx, j)
                    }
                    acc = mfma16<BF16>(acc, xo.v, so.v);
                }
                // lane: i = idx, c = c0 + 8 (r / 4) + 4 (lane / 32) + r % 4
                if(idx < m)
                {
#pragma unroll
                    for(uint32_t q = 0; q < 4; ++q)
                    {
                        union
                        {
                            uint16_t h[4];
                            uint64_t v;
                        } o;
#pragma unroll
                        for(uint32_t e = 0; e < 4; ++e)
                            o.h[e] = roundOut<BF16>(acc[4 * q + e]);
                        const uint32_t c = c0 + 8u * q + 4u * (lane >> 5);
                        *reinterpret_cast<uint64_t*>(inGrad + (uint64_t)b * m * K + idx * K + c) = o.v;
                    }
                }
            }
            __builtin_amdgcn_wave_barrier();
        }
    }

    int checkArgs(const char* what, int32_t dtype, const void* in, const void* out, uint32_t m, uint32_t k, uint32_t batch,
                  bool allowF32)
    {
        if(!in || !out)
            return r355::fail(R355_ERR_BAD_ARG, "%s: null pointer", what);
        if(dtype != R355_F16 && dtype != R355_BF16 && !(allowF32 && dtype == R355_F32))
            return r355::fail(R355_ERR_UNSUPPORTED, "%s: dtype must be R355_F16, R355_BF16%s", what, allowF32 ? " or R355_F32" : "");
        if(dtype == R355_F32 && k > 128)
            return r355::fail(R355_ERR_BAD_SIZE, "%s: k=%u must be at most 128 for R355_F32", what, k);
        if(m < 2 || m > MAX_M)
            return r355::fail(R355_ERR_BAD_SIZE, "%s: m=%u must be in [2, %u]", what, m, MAX_M);
        if(k != 32 && k != 64 && k != 128 && k != 256)
            return r355::fail(R355_ERR_BAD_SIZE, "%s: k=%u must be 32, 64, 128 or 256", what, k);
        if(batch == 0)
            return r355::fail(R355_ERR_BAD_ARG, "%s: batch is zero", what);
        if(!r355::aligned(in, 16) || !r355::aligned(out, 16))
            return r355::fail(R355_ERR_MISALIGNED, "%s: in / out must be 16-byte aligned", what);
        return R355_OK;
    }
} // namespace

extern "C" int r355_dlrm_fwd(int32_t dtype, const void* in, void* out, uint32_t m, uint32_t k, uint32_t batch, void* stream)
{
    int rc = checkArgs("dlrm_fwd", dtype, in, out, m, k, batch, true);
    if(rc != R355_OK)
        return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if(dtype == R355_F32)
    {
        const dim3 grid32((batch + WAVES - 1) / WAVES), block32(THREADS);
        auto*      fi = static_cast<const float*>(in);
        auto*      fo = static_cast<float*>(out);
        switch(k)
        {
        case 32: hipLaunchKernelGGL(dlrmFwdF32Kernel<32>, grid32, block32, 0, s, fi, fo, m, batch); break;
        case 64: hipLaunchKernelGGL(dlrmFwdF32Kernel<64>, grid32, block32, 0, s, fi, fo, m, batch); break;
        default: hipLaunchKernelGGL(dlrmFwdF32Kernel<128>, grid32, block32, 0, s, fi, fo, m, batch); break;
        }
        return r355::checkLaunch("dlrm_fwd");
    }
    const dim3 grid((batch + SAMPLES_PER_WG - 1) / SAMPLES_PER_WG), block(THREADS);
    auto*       pi = static_cast<const uint16_t*>(in);
    auto*       po = static_cast<uint16_t*>(out);
#define R355_FWD(BF, KK)                                                                         \
    do                                                                                            \
    {                                                                                             \
        if(m <= 28)                                                                               \
            hipLaunchKernelGGL((dlrmFwdKernel<BF, KK, 28>), grid, block, 0, s, pi, po, m, batch); \
        else                                                                                      \
            hipLaunchKernelGGL((dlrmFwdKernel<BF, KK, 32>), grid, block, 0, s, pi, po, m, batch); \
    } while(0)
#define R355_FWD_K(BF)   \
    switch(k)            \
    {                    \
    case 32: R355_FWD(BF, 32); break;   \
    case 64: R355_FWD(BF, 64); break;   \
    case 128: R355_FWD(BF, 128); break; \
    default: R355_FWD(BF, 256); break;  \
    }
    if(dtype == R355_BF16)
    {
        R355_FWD_K(true)
    }
    else
    {
        R355_FWD_K(false)
    }
#undef R355_FWD_K
#undef R355_FWD
    return r355::checkLaunch("dlrm_fwd");
}

extern "C" int r355_dlrm_bwd(int32_t dtype, const void* in, const void* upstream, void* mlp_grad, void* in_grad,
                             uint32_t m, uint32_t k, uint32_t batch, void* stream)
{
    int rc = checkArgs("dlrm_bwd", dtype, in, in_grad, m, k, batch, false);
    if(rc != R355_OK)
        return rc;
    if(!upstream || !mlp_grad)
        return r355::fail(R355_ERR_BAD_ARG, "dlrm_bwd: null pointer");
    const uint32_t wgs = (batch + WAVES - 1) / WAVES;
    const dim3     grid(wgs < 4096 ? wgs : 4096), block(THREADS);
    hipStream_t    s  = static_cast<hipStream_t>(stream);
    auto*          pi = static_cast<const uint16_t*>(in);
    auto*          pu = static_cast<const uint16_t*>(upstream);
    auto*          pm = static_cast<uint16_t*>(mlp_grad);
    auto*          pg = static_cast<uint16_t*>(in_grad);
#define R355_BWD(BF, KK) hipLaunchKernelGGL((dlrmBwdKernel<BF, KK>), grid, block, 0, s, pi, pu, pm, pg, m, batch)
#define R355_BWD_K(BF)   \
    switch(k)            \
    {                    \
    case 32: R355_BWD(BF, 32); break;   \
    case 64: R355_BWD(BF, 64); break;   \
    case 128: R355_BWD(BF, 128); break; \
    default: R355_BWD(BF, 256); break;  \
    }
    if(dtype == R355_BF16)
    {
        R355_BWD_K(true)
    }
    else
    {
        R355_BWD_K(false)
    }
#undef R355_BWD_K
#undef R355_BWD
    return r355::checkLaunch("dlrm_bwd");
}
