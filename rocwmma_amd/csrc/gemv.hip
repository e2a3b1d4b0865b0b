// GEMV y = alpha * A x + beta * y for f32 and f64, HBM-bound: A is read exactly once with
// coalesced 128-bit loads, x is staged through LDS, and f32 FMAs accumulate in the
// order k = 0..K-1 per output row within a lane.
//
// Takes the place of samples/simple_sgemv.cpp:103-150 (f64: samples/simple_dgemv.cpp:103), which feeds 16x16x16 f32 fragments
// (the B fragment being x broadcast 16 times) to the matrix core.  At 0.5 flop per byte
// the matrix core contributes nothing; the kernel is organised for memory bandwidth.
//   col-major A (the sample's layout): a workgroup owns 64 (or 256) rows; its 16 waves split
//     the columns and combine their partial sums through LDS in a fixed order.
//   row-major A: one wave per row, lanes stride k in float4, then a wave reduction.
#include <hip/hip_runtime.h>

#include "common.hpp"

namespace
{
    constexpr uint32_t THREADS = 256;

    // col-major A (m contiguous): a wave reads V * 64 consecutive rows of one column per load;
    // the 16 waves of a workgroup split the columns and their partial sums meet in LDS in a fixed
    // order, so the result does not depend on scheduling.
    constexpr uint32_t COL_WAVES = 16;

    template <typename T, uint32_t V>
    __global__ void __launch_bounds__(COL_WAVES * 64) gemvColMajor(uint32_t m,
                                                                  uint32_t k,
                                                                  const T* a,
                                                                  uint32_t lda,
                                                                  const T* x,
                                                                  const T* yIn,
                                                                  T*       yOut,
                                                                  T        alpha,
                                                                  T        beta)
    {
        using VecT = T __attribute__((ext_vector_type(V)));
        __shared__ T   partial[COL_WAVES][64 * V];
        const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
        const uint32_t r0   = (blockIdx.x * 64u + lane) * V;
        T              acc[V];
#pragma unroll
        for(uint32_t e = 0; e < V; ++e)
            acc[e] = T(0);
        if(r0 < m)
        {
            const T* p = a + r0;
#pragma unroll 8
            for(uint32_t kk = wave; kk < k; kk += COL_WAVES)
            {
                T v[V];
                if constexpr(V == 1)
                    v[0] = p[(uint64_t)kk * lda];
                else
                {
                    const VecT vv = *reinterpret_cast<const VecT*>(p + (uint64_t)kk * lda);
#pragma unroll
                    for(uint32_t e = 0; e < V; ++e)
                        v[e] = vv[e];
                }
                const T xv = x[kk];
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
                T sum = T(0);
#pragma unroll
                for(uint32_t w = 0; w < COL_WAVES; ++w)
                    sum += partial[w][r];
                yOut[row] = beta != T(0) ? alpha * sum + beta * yIn[row] : alpha * sum;
            }
        }
    }

    template <typename T>
    __global__ void __launch_bounds__(THREADS) gemvRowMajor(uint32_t m,
                                                           uint32_t k,
                                                           const T* a,
                                                           uint32_t lda,
                                                           const T* x,
                                                           const T* yIn,
                                                           T*       yOut,
                                                           T        alpha,
                                                           T        beta)
    {
        constexpr uint32_t V = 16u / sizeof(T); // elements of a 128-bit load
        using VecT           = T __attribute__((ext_vector_type(V)));
        const uint32_t lane  = threadIdx.x & 63u;
        const uint32_t row   = blockIdx.x * (THREADS / 64u) + threadIdx.x / 64u;
        if(row >= m)
            return;
        const T* p   = a + (uint64_t)row * lda;
        T        acc = T(0);
        for(uint32_t kk = lane * V; kk < k; kk += 64u * V)
        {
            const VecT v  = *reinterpret_cast<const VecT*>(p + kk);
            const VecT xv = *reinterpret_cast<const VecT*>(x + kk);
#pragma unroll
            for(uint32_t e = 0; e < V; ++e)
                acc += v[e] * xv[e];
        }
#pragma unroll
        for(uint32_t off = 32; off > 0; off >>= 1)
            acc += __shfl_xor(acc, off, 64);
        if(lane == 0)
            yOut[row] = beta != T(0) ? alpha * acc + beta * yIn[row] : alpha * acc;
    }

    template <typename T>
    int gemvLaunch(int32_t layout_a, uint32_t m, uint32_t k, const T* a, uint32_t lda, const T* x, const T* y_in, T* y_out,
                   T alpha, T beta, void* stream)
    {
        constexpr uint32_t V = 16u / sizeof(T);
        if(!a || !x || !y_out || (beta != T(0) && !y_in))
            return r355::fail(R355_ERR_BAD_ARG, "gemv: null pointer");
        if(m == 0 || k == 0)
            return r355::fail(R355_ERR_BAD_ARG, "gemv: m and k must be non-zero");
        if(m % V || k % V)
            return r355::fail(R355_ERR_BAD_SIZE, "gemv: m=%u and k=%u must be multiples of %u", m, k, V);
        if(!r355::aligned(a, 16) || lda % V || !r355::aligned(x, 16) || !r355::aligned(y_out, 16))
            return r355::fail(R355_ERR_MISALIGNED, "gemv: a, x, y need 16-byte alignment and lda %% %u == 0", V);
        hipStream_t s = static_cast<hipStream_t>(stream);
        if(layout_a == R355_COL_MAJOR)
        {
            if(lda < m)
                return r355::fail(R355_ERR_BAD_ARG, "gemv: lda < m");
            // narrow loads while they are what it takes to give every CU a workgroup
            if(m >= 64u * V * 256u)
                hipLaunchKernelGGL((gemvColMajor<T, V>), dim3((m + 64u * V - 1u) / (64u * V)), dim3(COL_WAVES * 64), 0, s, m, k, a,
                                   lda, x, y_in, y_out, alpha, beta);
            else
                hipLaunchKernelGGL((gemvColMajor<T, 1>), dim3((m + 63u) / 64u), dim3(COL_WAVES * 64), 0, s, m, k, a, lda, x,
                                   y_in, y_out, alpha, beta);
        }
        else if(layout_a == R355_ROW_MAJOR)
        {
            if(lda < k)
                return r355::fail(R355_ERR_BAD_ARG, "gemv: lda < k");
            hipLaunchKernelGGL((gemvRowMajor<T>), dim3((m + THREADS / 64 - 1) / (THREADS / 64)), dim3(THREADS), 0, s, m, k, a,
                               lda, x, y_in, y_out, alpha, beta);
        }
        else
            return r355::fail(R355_ERR_BAD_ARG, "gemv: unknown layout");
        return r355::checkLaunch("gemv");
    }
} // namespace

extern "C" int r355_gemv(int32_t layout_a, uint32_t m, uint32_t k, const float* a, uint32_t lda, const float* x,
                         const float* y_in, float* y_out, float alpha, float beta, void* stream)
{
    return gemvLaunch<float>(layout_a, m, k, a, lda, x, y_in, y_out, alpha, beta, stream);
}

extern "C" int r355_dgemv(int32_t layout_a, uint32_t m, uint32_t k, const double* a, uint32_t lda, const double* x,
                          const double* y_in, double* y_out, double alpha, double beta, void* stream)
{
    return gemvLaunch<double>(layout_a, m, k, a, lda, x, y_in, y_out, alpha, beta, stream);
}
