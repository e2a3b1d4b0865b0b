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
// Backward takes the place of test/dlrm/device/dlrm_dot_bwd.hpp:35-176: the symmetric matrix
// of the upstream triangle (trilReconstruct) is formed directly as a matrix-instruction operand
// and multiplied into X, read from LDS with transposing reads, again without global scratch.
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

    // f32 variant.  An f32 sample is 13.8 KB, so only a few fit in LDS per CU and the matrix core
    // (v_mfma_f32_16x16x4_f32, 96 instructions per sample) is busy a good third of the time: the loads
    // of a wave's next sample are therefore issued before the current sample is computed, and every
    // wave walks F32_PER_WAVE consecutive samples, writing each result row from its own LDS image
    // with coalesced 4-byte stores (a sample's output row is only 4-byte aligned).
    constexpr uint32_t F32_PER_WAVE = 8;

    template <uint32_t K, uint32_t ROWS>
    __global__ void __launch_bounds__(THREADS)
        dlrmFwdF32Kernel(const float* __restrict__ in, float* __restrict__ out, uint32_t m, uint32_t batch)
    {
        constexpr uint32_t ROW_CHUNKS = K / 4; // 16-byte chunks per row
        constexpr uint32_t MAX_OUT    = K + ROWS * (ROWS - 1) / 2;
        constexpr uint32_t MAX_CHUNKS = (ROWS * ROW_CHUNKS + 63u) / 64u;
        constexpr uint32_t SWZ        = 31u & (ROW_CHUNKS - 1u);
        using f32x4                   = float __attribute__((ext_vector_type(4)));

        __shared__ __attribute__((aligned(16))) float xLds[WAVES][ROWS * K];
        __shared__ __attribute__((aligned(16))) float outLds[WAVES][MAX_OUT];

        const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
        const uint32_t outStride = K + m * (m - 1) / 2;
        const uint32_t inChunks  = m * ROW_CHUNKS;
        const uint32_t first     = (blockIdx.x * WAVES + wave) * F32_PER_WAVE; // this wave's first sample
        char*          xw        = reinterpret_cast<char*>(xLds[wave]);
        float*         o         = outLds[wave];

        f32x4 stash[2][MAX_CHUNKS];
        auto  request = [&](uint32_t b, f32x4 (&dst)[MAX_CHUNKS]) {
            if(b < batch)
            {
                const char* src = reinterpret_cast<const char*>(in) + (uint64_t)b * m * K * 4u;
#pragma unroll
                for(uint32_t j = 0; j < MAX_CHUNKS; ++j)
                {
                    const uint32_t c = j * 64u + lane;
                    if(c < inChunks)
                        dst[j] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(src + c * 16u));
                }
            }
        };
        auto process = [&](uint32_t b, const f32x4 (&src)[MAX_CHUNKS]) {
            if(b >= batch)
                return;
#pragma unroll
            for(uint32_t j = 0; j < MAX_CHUNKS; ++j)
            {
                const uint32_t c = j * 64u + lane;
                if(c < inChunks)
                {
                    const uint32_t row = c / ROW_CHUNKS, col = c % ROW_CHUNKS;
                    *reinterpret_cast<f32x4*>(xw + (row * ROW_CHUNKS + (col ^ (row & SWZ))) * 16u) = src[j];
                }
            }
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __builtin_amdgcn_wave_barrier();

            // v_mfma_f32_16x16x4_f32 on the three 16 x 16 blocks of the Gram matrix that hold its lower
            // triangle (rows < 16 x rows < 16, rows >= 16 x rows < 16, rows >= 16 x rows >= 16): a quarter
            // fewer matrix-core cycles than the full 32 x 32 product, and three independent accumulator
            // chains keep the pipeline full.  Lane l feeds row l % 16 (+ 16) at k = 4 s + l / 16.
            using f32x4acc = float __attribute__((ext_vector_type(4)));
            f32x4acc       accLL = {0, 0, 0, 0}, accHL = accLL, accHH = accLL;
            const uint32_t r16 = lane & 15u, kq = lane >> 4;
            const bool     validLo = r16 < m, validHi = 16u + r16 < m;
            const uint32_t rowLo = validLo ? r16 : 0u, rowHi = validHi ? 16u + r16 : 0u;
#pragma unroll 8
            for(uint32_t s = 0; s < K / 4; ++s)
            {
                float xl = *reinterpret_cast<const float*>(xw + (rowLo * ROW_CHUNKS + (s ^ (rowLo & SWZ))) * 16u + kq * 4u);
                float xh = *reinterpret_cast<const float*>(xw + (rowHi * ROW_CHUNKS + (s ^ (rowHi & SWZ))) * 16u + kq * 4u);
                if(!validLo)
                    xl = 0.0f;
                if(!validHi)
                    xh = 0.0f;
                accLL = __builtin_amdgcn_mfma_f32_16x16x4f32(xl, xl, accLL, 0, 0, 0);
                accHL = __builtin_amdgcn_mfma_f32_16x16x4f32(xh, xl, accHL, 0, 0, 0);
                accHH = __builtin_amdgcn_mfma_f32_16x16x4f32(xh, xh, accHH, 0, 0, 0);
            }

            for(uint32_t e = lane; e < K; e += 64)
                o[e] = reinterpret_cast<const float*>(xw)[e]; // row 0 is stored unswizzled
            // a 16 x 16 result block: lane holds rows 4 (lane / 16) + e, column lane % 16
#pragma unroll
            for(uint32_t e = 0; e < 4; ++e)
            {
                const uint32_t i = 4u * kq + e, j = r16;
                if(j < i && i < m)
                    o[K + i * (i - 1u) / 2u + j] = accLL[e];
                const uint32_t ih = 16u + i;
                if(ih < m)
                {
                    o[K + ih * (ih - 1u) / 2u + j] = accHL[e];
                    if(j < i)
                        o[K + ih * (ih - 1u) / 2u + 16u + j] = accHH[e];
                }
            }
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __builtin_amdgcn_wave_barrier();
            float* dst = out + (uint64_t)b * outStride;
            for(uint32_t e = lane; e < outStride; e += 64)
                __builtin_nontemporal_store(o[e], dst + e);
            __builtin_amdgcn_s_waitcnt(0xC07F); // the image is rewritten by the next sample
            __builtin_amdgcn_wave_barrier();
        };

        request(first, stash[0]);
#pragma unroll 1
        for(uint32_t it = 0; it < F32_PER_WAVE; it += 2)
        {
            request(first + it + 1u, stash[1]);
            process(first + it, stash[0]);
            if(it + 2u < F32_PER_WAVE)
                request(first + it + 2u, stash[0]);
            process(first + it + 1u, stash[1]);
        }
    }

    // Backward: S = T + T^T (T = strict lower triangle from the upstream gradient, zero diagonal),
    // grad (m x k) = S X.  Same organisation as the forward kernel: a workgroup owns 8 consecutive
    // samples (their upstream rows form one 16-byte aligned run, staged in LDS with 128-bit loads),
    // a wave owns one sample at a time with the X of both of its samples requested up front.
    // X sits in LDS as [j][c] rows; the matrix instruction wants X^T (lane = column c, 8
    // consecutive j), which the transposing LDS read delivers: 16 lanes address a 4 (j) x 16 (c)
    // block and lane t receives column t.  Per 32-column slab of k: acc(c, i) = sum_j X(j, c) S(j, i),
    // i.e. every lane ends up with runs of 4 consecutive c of one gradient row i.  The gradient
    // image replaces X in LDS (rows < m) and leaves with 128-bit nontemporal stores.
    typedef __fp16 trv4 __attribute__((__vector_size__(4 * sizeof(__fp16))));

    template <bool BF16, uint32_t K, uint32_t ROWS>
    __global__ void __launch_bounds__(THREADS) dlrmBwdKernel(const uint16_t* __restrict__ in,
                                                            const uint16_t* __restrict__ upstream,
                                                            uint16_t* __restrict__ mlpGrad,
                                                            uint16_t* __restrict__ inGrad,
                                                            uint32_t m,
                                                            uint32_t batch)
    {
        constexpr uint32_t ROW_CHUNKS = K / 8; // 16-byte chunks per row
        constexpr uint32_t ROWB       = K * 2;
        constexpr uint32_t X_BYTES    = MAX_M * ROWB; // always 32 rows: rows >= m stay zero
        constexpr uint32_t SLABS      = K / 32;
        constexpr uint32_t MAX_UP     = K + ROWS * (ROWS - 1) / 2;
        constexpr uint32_t PER_WAVE   = SAMPLES_PER_WG / WAVES;
        constexpr uint32_t MAX_CHUNKS = (ROWS * ROW_CHUNKS + 63u) / 64u;
        constexpr uint32_t SWZ_IN     = 12u & (ROW_CHUNKS - 1u); // (j & 3) << 2: four j rows -> four 64-byte groups
        constexpr uint32_t SWZ_OUT    = 15u & (ROW_CHUNKS - 1u);

        __shared__ __attribute__((aligned(16))) char     xLds[WAVES][X_BYTES];
        __shared__ __attribute__((aligned(16))) uint16_t upLds[SAMPLES_PER_WG * MAX_UP + 8];

        const uint32_t tid      = threadIdx.x;
        const uint32_t lane     = tid & 63u;
        const uint32_t wave     = tid >> 6;
        const uint32_t upStride = K + m * (m - 1) / 2;
        const uint32_t b0       = blockIdx.x * SAMPLES_PER_WG;
        const uint32_t inChunks = m * ROW_CHUNKS;
        char*          xw       = xLds[wave];

        i32x4 stash[PER_WAVE][MAX_CHUNKS];
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
                        stash[q][j] = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(src + c * 16u));
                }
            }
        }

        // ---- upstream rows of the workgroup's samples -> LDS; zero rows m..31 of the X image
        const uint32_t nSamples = (batch - b0) < SAMPLES_PER_WG ? (batch - b0) : SAMPLES_PER_WG;
        {
            const uint32_t  total = nSamples * upStride;
            const uint16_t* src   = upstream + (uint64_t)b0 * upStride;
            const uint32_t  vecs  = total / 8u;
            for(uint32_t v = tid; v < vecs; v += THREADS)
                reinterpret_cast<i32x4*>(upLds)[v] = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(src) + v);
            for(uint32_t e = vecs * 8u + tid; e < total; e += THREADS)
                upLds[e] = src[e];
            for(uint32_t c = inChunks + lane; c < MAX_M * ROW_CHUNKS; c += 64u)
                *reinterpret_cast<i32x4*>(xw + c * 16u) = i32x4{0, 0, 0, 0};
        }
        __syncthreads();

        // ---- bottom-MLP gradient: the first k values of every upstream row
        for(uint32_t t = tid; t < nSamples * ROW_CHUNKS; t += THREADS)
        {
            const uint32_t sIdx = t / ROW_CHUNKS, cc = t % ROW_CHUNKS;
            union
            {
                uint16_t h[8];
                i32x4    v;
            } o;
#pragma unroll
            for(uint32_t e = 0; e < 8; ++e)
                o.h[e] = upLds[sIdx * upStride + cc * 8u + e];
            __builtin_nontemporal_store(o.v, reinterpret_cast<i32x4*>(mlpGrad + ((uint64_t)(b0 + sIdx) * K + cc * 8u)));
        }

        const uint32_t i = lane & 31u, half = lane >> 5, t16 = lane & 15u;
#pragma unroll
        for(uint32_t q = 0; q < PER_WAVE; ++q)
        {
            const uint32_t sIdx = wave + q * WAVES;
            const uint32_t b    = b0 + sIdx;
            if(b >= batch)
                break;
            // ---- X -> LDS: chunk c goes to row j = c / ROW_CHUNKS, slot (c % ROW_CHUNKS) ^ ((j & 3) << 2)
#pragma unroll
            for(uint32_t j = 0; j < MAX_CHUNKS; ++j)
            {
                const uint32_t c = j * 64u + lane;
                if(c < inChunks)
                {
                    const uint32_t row = c / ROW_CHUNKS, col = c % ROW_CHUNKS;
                    *reinterpret_cast<i32x4*>(xw + (row * ROW_CHUNKS + (col ^ ((row << 2) & SWZ_IN))) * 16u) = stash[q][j];
                }
            }
            // ---- S operand: lane holds S(i, j) for its 8-wide runs of j (zero diagonal, zero padding)
            const uint16_t* tril = upLds + sIdx * upStride + K;
            i32x4           sReg[2];
#pragma unroll
            for(uint32_t s = 0; s < 2; ++s)
            {
                union
                {
                    uint16_t h[8];
                    i32x4    v;
                } so;
#pragma unroll
                for(uint32_t e = 0; e < 8; ++e)
                {
                    const uint32_t j  = 16u * s + 8u * half + e;
                    const uint32_t hi = i > j ? i : j, lo = i > j ? j : i;
                    uint16_t       v  = 0;
                    if(hi < m && hi != lo)
                        v = tril[hi * (hi - 1u) / 2u + lo];
                    so.h[e] = v;
                }
                sReg[s] = so.v;
            }
            __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0): this wave's LDS writes are done
            __builtin_amdgcn_wave_barrier();

            f32x16 acc[SLABS];
#pragma unroll
            for(uint32_t slab = 0; slab < SLABS; ++slab)
            {
                acc[slab] = f32x16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
                for(uint32_t s = 0; s < 2; ++s)
                {
                    using lp             = __attribute__((address_space(3))) trv4*;
                    const uint32_t row   = 16u * s + 8u * half + (t16 >> 2);
                    const uint32_t piece = 8u * slab + 4u * ((lane >> 4) & 1u) + (t16 & 3u); // 8-byte pieces
                    const char*    p0    = xw + row * ROWB + (((piece >> 1) ^ ((row << 2) & SWZ_IN)) * 16u) + (piece & 1u) * 8u;
                    using i32x2          = int __attribute__((ext_vector_type(2)));
                    const i32x2 lo = __builtin_bit_cast(i32x2, __builtin_amdgcn_ds_read_tr16_b64_v4f16((lp)p0));
                    const i32x2 hi = __builtin_bit_cast(i32x2, __builtin_amdgcn_ds_read_tr16_b64_v4f16((lp)(p0 + 4u * ROWB)));
                    acc[slab]      = mfma16<BF16>(acc[slab], i32x4{lo[0], lo[1], hi[0], hi[1]}, sReg[s]);
                }
            }
            __builtin_amdgcn_s_waitcnt(0xC07F); // every read of X has returned before rows are overwritten
            __builtin_amdgcn_wave_barrier();

            // ---- gradient image over rows < m: lane has c = 32 slab + 8 r + 4 half + (0..3) of row i
            if(i < m)
            {
#pragma unroll
                for(uint32_t slab = 0; slab < SLABS; ++slab)
#pragma unroll
                    for(uint32_t r = 0; r < 4; ++r)
                    {
                        union
                        {
                            uint16_t h[4];
                            uint64_t v;
                        } o;
#pragma unroll
                        for(uint32_t e = 0; e < 4; ++e)
                            o.h[e] = roundOut<BF16>(acc[slab][4 * r + e]);
                        const uint32_t chunk = 4u * slab + r;
                        *reinterpret_cast<uint64_t*>(xw + i * ROWB + ((chunk ^ (i & SWZ_OUT)) * 16u) + half * 8u) = o.v;
                    }
            }
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __builtin_amdgcn_wave_barrier();

            char* dst = reinterpret_cast<char*>(inGrad) + (uint64_t)b * m * K * 2u;
#pragma unroll
            for(uint32_t j = 0; j < MAX_CHUNKS; ++j)
            {
                const uint32_t c = j * 64u + lane;
                if(c < inChunks)
                {
                    const uint32_t row = c / ROW_CHUNKS, col = c % ROW_CHUNKS;
                    const i32x4    v   = *reinterpret_cast<const i32x4*>(xw + (row * ROW_CHUNKS + (col ^ (row & SWZ_OUT))) * 16u);
                    __builtin_nontemporal_store(v, reinterpret_cast<i32x4*>(dst + c * 16u));
                }
            }
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __builtin_amdgcn_wave_barrier();
        }
    }

    // f32 backward.  grad (m x k) = S X with S = T + T^T from the upstream triangle, on
    // v_mfma_f32_16x16x4_f32: A operand = a 16 x 4 piece of S (lane l: row l % 16, column l / 16), B
    // operand = a 4 x 16 piece of X (lane l: row l / 16, column l % 16), 2 x (k / 16) result blocks, 8
    // steps over the 32 (zero-padded) rows of X.  Every wave walks F32_PER_WAVE consecutive samples with
    // the loads of the next one in flight.  Per sample: X goes to an LDS image whose 64-byte column
    // groups are XOR-swizzled with the row (four consecutive rows of one column group land in
    // different banks), the upstream row to a second image from which each lane gathers its 16 values
    // of S; the gradient is written over X and leaves with 128-bit nontemporal stores; the first k
    // upstream values are the bottom-MLP gradient (test/reference_impl.hpp:121-179).
    template <uint32_t K>
    __global__ void __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(2))) dlrmBwdF32Kernel(const float* __restrict__ in, const float* __restrict__ upstream,
                                                               float* __restrict__ mlpGrad, float* __restrict__ inGrad,
                                                               uint32_t m, uint32_t batch)
    {
        constexpr uint32_t ROW_CHUNKS = K / 4; // 16-byte chunks per row
        constexpr uint32_t ROWB       = K * 4;
        constexpr uint32_t MAX_UP     = K + MAX_M * (MAX_M - 1) / 2;
        constexpr uint32_t X_CHUNKS   = (MAX_M * ROW_CHUNKS + 63u) / 64u; // per lane
        constexpr uint32_t UP_WORDS   = (MAX_UP + 63u) / 64u; // per lane
        constexpr uint32_t CBLOCKS    = K / 16; // 64-byte column groups per row
        constexpr uint32_t SWZ        = CBLOCKS >= 4 ? 3u : CBLOCKS - 1u;
        using f32x4                   = float __attribute__((ext_vector_type(4)));

        __shared__ __attribute__((aligned(16))) char  xLds[WAVES][MAX_M * ROWB];
        __shared__ __attribute__((aligned(16))) float upLds[WAVES][MAX_UP];

        const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
        const uint32_t upStride = K + m * (m - 1) / 2;
        const uint32_t inChunks = m * ROW_CHUNKS;
        const uint32_t first    = (blockIdx.x * WAVES + wave) * F32_PER_WAVE;
        char*          xw       = xLds[wave];
        float*         uw       = upLds[wave];
        const uint32_t r16 = lane & 15u, q4 = lane >> 4;

        // byte address of 16-byte chunk c (0 .. ROW_CHUNKS) of row `row` in the swizzled image
        auto chunkAt = [&](uint32_t row, uint32_t c) { return row * ROWB + ((((c >> 2) ^ (row & SWZ)) << 2) + (c & 3u)) * 16u; };

        // rows >= m of the image stay zero for every sample
        for(uint32_t c = inChunks + lane; c < MAX_M * ROW_CHUNKS; c += 64u)
            *reinterpret_cast<f32x4*>(xw + chunkAt(c / ROW_CHUNKS, c % ROW_CHUNKS)) = f32x4{0, 0, 0, 0};

        // where lane l finds S(i, j) in the upstream image: the strict lower triangle is stored row by
        // row behind the first k values; the diagonal is zero (recomputed per sample: registers are
        // scarcer than integer instructions here)
        auto sAt = [&](uint32_t i, uint32_t j) -> float {
            const uint32_t hi = i > j ? i : j, lo = i > j ? j : i;
            return (i != j && hi < m) ? uw[K + hi * (hi - 1u) / 2u + lo] : 0.0f;
        };

        // one register stash: a sample's loads are requested while the previous sample is computed and
        // unloaded into LDS before the next request reuses the registers
        f32x4 xs[X_CHUNKS];
        float us[UP_WORDS];
        auto  request = [&](uint32_t b) {
            if(b < batch)
            {
                const char*  src = reinterpret_cast<const char*>(in) + (uint64_t)b * m * ROWB;
                const float* up  = upstream + (uint64_t)b * upStride;
#pragma unroll
                for(uint32_t j = 0; j < X_CHUNKS; ++j)
                    if(j * 64u + lane < inChunks)
                        xs[j] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(src + (j * 64u + lane) * 16u));
#pragma unroll
                for(uint32_t j = 0; j < UP_WORDS; ++j)
                    if(j * 64u + lane < upStride)
                        us[j] = __builtin_nontemporal_load(up + j * 64u + lane);
            }
        };

        request(first);
#pragma unroll 1
        for(uint32_t it = 0; it < F32_PER_WAVE; ++it)
        {
            const uint32_t b = first + it;
            if(b >= batch)
                break;
#pragma unroll
            for(uint32_t j = 0; j < X_CHUNKS; ++j)
            {
                const uint32_t c = j * 64u + lane;
                if(c < inChunks)
                    *reinterpret_cast<f32x4*>(xw + chunkAt(c / ROW_CHUNKS, c % ROW_CHUNKS)) = xs[j];
            }
#pragma unroll
            for(uint32_t j = 0; j < UP_WORDS; ++j)
                if(j * 64u + lane < upStride)
                    uw[j * 64u + lane] = us[j];
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __builtin_amdgcn_wave_barrier();
            if(it + 1u < F32_PER_WAVE)
                request(b + 1u);

            // bottom-MLP gradient: the first k upstream values
            float* mg = mlpGrad + (uint64_t)b * K;
            for(uint32_t e = lane; e < K; e += 64u)
                __builtin_nontemporal_store(uw[e], mg + e);

            float sv[2][8];
#pragma unroll
            for(uint32_t ib = 0; ib < 2; ++ib)
#pragma unroll
                for(uint32_t js = 0; js < 8; ++js)
                    sv[ib][js] = sAt(16u * ib + r16, 4u * js + q4);

            f32x4 acc[2][CBLOCKS];
#pragma unroll
            for(uint32_t ib = 0; ib < 2; ++ib)
#pragma unroll
                for(uint32_t cb = 0; cb < CBLOCKS; ++cb)
                    acc[ib][cb] = f32x4{0, 0, 0, 0};
#pragma unroll
            for(uint32_t js = 0; js < 8; ++js)
            {
                const uint32_t row = 4u * js + q4;
#pragma unroll
                for(uint32_t cb = 0; cb < CBLOCKS; ++cb)
                {
                    // X(row, 16 cb + l % 16): 64-byte column group cb, swizzled with the row
                    const float xv = *reinterpret_cast<const float*>(xw + row * ROWB + ((cb ^ (row & SWZ)) << 6) + r16 * 4u);
                    acc[0][cb]     = __builtin_amdgcn_mfma_f32_16x16x4f32(sv[0][js], xv, acc[0][cb], 0, 0, 0);
                    acc[1][cb]     = __builtin_amdgcn_mfma_f32_16x16x4f32(sv[1][js], xv, acc[1][cb], 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0); // keeps the LDS reads of later steps from piling up in registers
            }
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __builtin_amdgcn_wave_barrier(); // every lane has read X: the gradient goes over it
            // result block (ib, cb): lane holds rows 16 ib + 4 (l / 16) + e, column 16 cb + l % 16
#pragma unroll
            for(uint32_t ib = 0; ib < 2; ++ib)
#pragma unroll
                for(uint32_t cb = 0; cb < CBLOCKS; ++cb)
#pragma unroll
                    for(uint32_t e = 0; e < 4; ++e)
                    {
                        const uint32_t row = 16u * ib + 4u * q4 + e;
                        if(row < m)
                            *reinterpret_cast<float*>(xw + row * ROWB + ((cb ^ (row & SWZ)) << 6) + r16 * 4u) = acc[ib][cb][e];
                    }
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __builtin_amdgcn_wave_barrier();
            char* dst = reinterpret_cast<char*>(inGrad) + (uint64_t)b * m * ROWB;
#pragma unroll
            for(uint32_t j = 0; j < X_CHUNKS; ++j)
            {
                const uint32_t c = j * 64u + lane;
                if(c < inChunks)
                    __builtin_nontemporal_store(*reinterpret_cast<const f32x4*>(xw + chunkAt(c / ROW_CHUNKS, c % ROW_CHUNKS)),
                                                reinterpret_cast<f32x4*>(dst + c * 16u));
            }
            __builtin_amdgcn_s_waitcnt(0xC07F); // the images are rewritten by the next sample
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
        const uint32_t perWg = WAVES * F32_PER_WAVE;
        const dim3     grid32((batch + perWg - 1) / perWg), block32(THREADS);
        auto*      fi = static_cast<const float*>(in);
        auto*      fo = static_cast<float*>(out);
#define R355_FWD32(KK)                                                                                \
    do                                                                                                \
    {                                                                                                 \
        if(m <= 28)                                                                                   \
            hipLaunchKernelGGL((dlrmFwdF32Kernel<KK, 28>), grid32, block32, 0, s, fi, fo, m, batch);  \
        else                                                                                          \
            hipLaunchKernelGGL((dlrmFwdF32Kernel<KK, 32>), grid32, block32, 0, s, fi, fo, m, batch);  \
    } while(0)
        switch(k)
        {
        case 32: R355_FWD32(32); break;
        case 64: R355_FWD32(64); break;
        default: R355_FWD32(128); break;
        }
#undef R355_FWD32
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
    int rc = checkArgs("dlrm_bwd", dtype, in, in_grad, m, k, batch, true);
    if(rc != R355_OK)
        return rc;
    if(!upstream || !mlp_grad)
        return r355::fail(R355_ERR_BAD_ARG, "dlrm_bwd: null pointer");
    if(dtype == R355_F32)
    {
        if(!r355::aligned(upstream, 4) || !r355::aligned(mlp_grad, 4))
            return r355::fail(R355_ERR_MISALIGNED, "dlrm_bwd: upstream and mlp_grad must be 4-byte aligned");
        const uint32_t perWg = WAVES * F32_PER_WAVE;
        const dim3     grid32((batch + perWg - 1) / perWg), block32(THREADS);
        hipStream_t    s32 = static_cast<hipStream_t>(stream);
        auto*          fi  = static_cast<const float*>(in);
        auto*          fu  = static_cast<const float*>(upstream);
        auto*          fm  = static_cast<float*>(mlp_grad);
        auto*          fg  = static_cast<float*>(in_grad);
        switch(k)
        {
        case 32: hipLaunchKernelGGL(dlrmBwdF32Kernel<32>, grid32, block32, 0, s32, fi, fu, fm, fg, m, batch); break;
        case 64: hipLaunchKernelGGL(dlrmBwdF32Kernel<64>, grid32, block32, 0, s32, fi, fu, fm, fg, m, batch); break;
        default: hipLaunchKernelGGL(dlrmBwdF32Kernel<128>, grid32, block32, 0, s32, fi, fu, fm, fg, m, batch); break;
        }
        return r355::checkLaunch("dlrm_bwd");
    }
    if(!r355::aligned(upstream, 16) || !r355::aligned(mlp_grad, 16))
        return r355::fail(R355_ERR_MISALIGNED, "dlrm_bwd: upstream and mlp_grad must be 16-byte aligned");
    const dim3  grid((batch + SAMPLES_PER_WG - 1) / SAMPLES_PER_WG), block(THREADS);
    hipStream_t s  = static_cast<hipStream_t>(stream);
    auto*       pi = static_cast<const uint16_t*>(in);
    auto*       pu = static_cast<const uint16_t*>(upstream);
    auto*       pm = static_cast<uint16_t*>(mlp_grad);
    auto*       pg = static_cast<uint16_t*>(in_grad);
#define R355_BWD(BF, KK)                                                                                          \
    do                                                                                                            \
    {                                                                                                             \
        if(m <= 28)                                                                                               \
            hipLaunchKernelGGL((dlrmBwdKernel<BF, KK, 28>), grid, block, 0, s, pi, pu, pm, pg, m, batch);          \
        else                                                                                                      \
            hipLaunchKernelGGL((dlrmBwdKernel<BF, KK, 32>), grid, block, 0, s, pi, pu, pm, pg, m, batch);          \
    } while(0)
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
        R355_BWD_K(true);
    }
    else
    {
        R355_BWD_K(false);
    }
#undef R355_BWD_K
#undef R355_BWD
    return r355::checkLaunch("dlrm_bwd");
}
