// Runs the device kernel of the reference's samples/simple_dgemm.cpp, compiled unchanged against
// this library's headers, with the sample's own launch geometry (samples/simple_dgemm.cpp:186-218).
#define main sample_main_unused
#include "simple_dgemm.cpp"
#undef main

extern "C" int ref_simple_dgemm(uint32_t m, uint32_t n, uint32_t k, const void* a, const void* b, const void* c, void* d,
                                uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd, double alpha, double beta)
{
    using T = rocwmma::float64_t;
    auto blockDim = dim3(4 * 64, T_BLOCK_Y);
    auto gridDim  = dim3(rocwmma::ceilDiv(m, ROCWMMA_M * 4u), rocwmma::ceilDiv(n, ROCWMMA_N * T_BLOCK_Y));
    hipLaunchKernelGGL(dgemm_rocwmma_d, gridDim, blockDim, 0, 0, m, n, k, static_cast<const T*>(a),
                       static_cast<const T*>(b), static_cast<const T*>(c), static_cast<T*>(d), lda, ldb, ldc, ldd,
                       static_cast<T>(alpha), static_cast<T>(beta));
    return hipDeviceSynchronize() == hipSuccess ? 0 : -1;
}
