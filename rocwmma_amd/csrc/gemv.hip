// GEMV y = alpha * A x + beta * y for f32, HBM-bound: A is read exactly once with
// coalesced 128-bit loads, x is staged through LDS, and f32 FMAs accumulate in the
// order k = 0..K-1 per output row within a lane.
//
// Takes the place of samples/simple_sgemv.cpp:103-150, which feeds 16x16x16 f32 fragments
// (the B fragment being x broadcast 16 times) to the matrix core.  At 0.5 flop per byte
// the matrix core contributes nothing; the kernel is organised for memory bandwidth.
//   col-major A (the sample's layout): a workgroup owns 64 (or 256) rows; its 16 waves split
//     the columns and combine their partial sums through LDS in a fixed order.
//   row-major A: one wave per row, lanes stride k in float4, then a wave reduction.
#include <hip/hip_runtime.h>

#include "common.hpp"

namespace
{
    using f32x4 = float __attribute__((ext_vector_type(4)));

    constexpr uint32_t THREADS = 256;

    // col-major A (m contiguous): a wave reads V * 64 consecutive rows of one column per load;
    // the 16 waves of a workgroup split the columns and their partial sums meet in LDS in a fixed
    // order, so the result does not depend on scheduling.
    constexpr uint32_t COL_WAVES = 16;

    template <uint32_t V>
    __global__ void __launch_bounds__(COL_WAVES * 64) gemvColMajor(uint32_t     m,
                                                                  uint32_t     k,
                                                                  const float* a,
                                                                  uint32_t     lda,
                                                                  const float* x,
                                                                  const float* yIn,
                                                                  float*       yOut,
                                                                  float        alpha,
                                                                  float        beta)
    {
        using VecT = float __attribute__((ext_vector_type(V)));
        __shared__ float partial[COL_WAVES][64 * V];
        const uint32_t   lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
        const uint32_t   r0   = (blockIdx.x * 64u + lane) * V;
        VecT             acc;
#pragma unroll
        for(uint32_t e = 0; e < V; ++e)
            acc[e] = 0.0f;
        if(r0 < m)
        {
            const float* p = a + r0;
#pragma unroll 8
            for(uint32_t kk = wave; kk < k; kk += COL_WAVES)
            {
                const VecT  v  = *reinterpret_cast<const VecT*>(p + (uint64_t)kk * lda);
                const float xv = x[kk];
#pragma unroll
                for(uint32_t e = 0; e < V; ++e)
                    acc[e] += v[e] * xv;
            }
        }
#pragma unroll
        for(uint32_t e = 0; e < V; ++e)
            partial[wave][lane * V + e] = acc[e];
        __syncthreads();
        // 64 * V rows, summed over the waves in wave order
        for(uint32_t r = threadIdx.x; r < 64u * V; r += COL_WAVES * 64u)
        {
            const uint32_t row = blockIdx.x * 64u * V + r;
            if(row < m)
            {
                float sum = 0.0f;
#pragma unroll
                for(uint32_t w = 0; w < COL_WAVES; ++w)
                    sum += partial[w][r];
                yOut[row] = beta != 0.0f ? alpha * sum + beta * yIn[row] : alpha * sum;
            }
        }
    }

    __global__ void __launch_bounds__(THREADS) gemvRowMajor(uint32_t     m,
                                                           uint32_t     k,
                                                           const float* a,
                                                           uint32_t     lda,
                                                           const float* x,
                                                           const float* yIn,
                                                           float*       yOut,
                                                           float        alpha,
                                                           float        beta)
    {
        const uint32_t lane = threadIdx.x & 63u;
        const uint32_t row  = blockIdx.x * (THREADS / 64u) + threadIdx.x / 64u;
        if(row >= m)
            return;
        const float* p   = a + (uint64_t)row * lda;
        float        acc = 0.0f;
        for(uint32_t kk = lane * 4u; kk < k; kk += 256u)
        {
            const f32x4 v  = *reinterpret_cast<const f32x4*>(p + kk);
            const f32x4 xv = *reinterpret_cast<const f32x4*>(x + kk);
            acc += v[0] * xv[0];
            acc += v[1] * xv[1];
            acc += v[2] * xv[2];
            acc += v[3] * xv[3];
        }
#pragma unroll
        for(uint32_t off = 32; off > 0; off >>= 1)
            acc += __shfl_xor(acc, off, 64);
        if(lane == 0)
            yOut[row] = beta != 0.0f ? alpha * acc + beta * yIn[row] : alpha * acc;
    }
} // namespace

extern "C" int r355_gemv(int32_t layout_a, uint32_t m, uint32_t k, const float* a, uint32_t lda, const float* x,
                         const float* y_in, float* y_out, float alpha, float beta, void* stream)
{
    if(!a || !x || !y_out || (beta != 0.0f && !y_in))
        return r355::fail(R355_ERR_BAD_ARG, "gemv: null pointer");
    if(m == 0 || k == 0)
        return r355::fail(R355_ERR_BAD_ARG, "gemv: m and k must be non-zero");
    if(m % 4 || k % 4)
        return r355::fail(R355_ERR_BAD_SIZE, "gemv: m=%u and k=%u must be multiples of 4", m, k);
    if(!r355::aligned(a, 16) || lda % 4 || !r355::aligned(x, 16) || !r355::aligned(y_out, 16))
        return r355::fail(R355_ERR_MISALIGNED, "gemv: a, x, y need 16-byte alignment and lda %% 4 == 0");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if(layout_a == R355_COL_MAJOR)
    {
        if(lda < m)
            return r355::fail(R355_ERR_BAD_ARG, "gemv: lda < m");
        // narrow loads while they are what it takes to give every CU a workgroup
        if(m >= 256u * 256u)
            hipLaunchKernelGGL(gemvColMajor<4>, dim3((m + 255u) / 256u), dim3(COL_WAVES * 64), 0, s, m, k, a, lda, x,
                               y_in, y_out, alpha, beta);
        else
            hipLaunchKernelGGL(gemvColMajor<1>, dim3((m + 63u) / 64u), dim3(COL_WAVES * 64), 0, s, m, k, a, lda, x,
                               y_in, y_out, alpha, beta);
    }
    else if(layout_a == R355_ROW_MAJOR)
    {
        if(lda < k)
            return r355::fail(R355_ERR_BAD_ARG, "gemv: lda < k");
        hipLaunchKernelGGL(gemvRowMajor, dim3((m + THREADS / 64 - 1) / (THREADS / 64)), dim3(THREADS), 0, s, m, k, a,
                           lda, x, y_in, y_out, alpha, beta);
    }
    else
        return r355::fail(R355_ERR_BAD_ARG, "gemv: unknown layout");
    return r355::checkLaunch("gemv");
}
