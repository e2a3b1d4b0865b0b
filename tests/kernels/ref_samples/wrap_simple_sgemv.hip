// Runs the device kernel of the reference's samples/simple_sgemv.cpp, compiled unchanged against this
// library's headers, with the sample's launch geometry (samples/simple_sgemv.cpp:198-226).
#define main sample_main_unused
#include "simple_sgemv.cpp"
#undef main

extern "C" int ref_simple_sgemv(uint32_t m, uint32_t n, uint32_t k, const float* a, const float* b, float* c, uint32_t lda,
                                uint32_t ldb, uint32_t ldc, uint32_t ldd, float alpha, float beta)
{
    auto blockDim = dim3(16 * 64, T_BLOCK_Y);
    auto gridDim  = dim3(rocwmma::ceilDiv(m, ROCWMMA_M * 16u), rocwmma::ceilDiv(n, ROCWMMA_N * T_BLOCK_Y));
    hipLaunchKernelGGL(sgemv_rocwmma_d, gridDim, blockDim, 0, 0, m, n, k, a, b, c, c, lda, ldb, ldc, ldd, alpha, beta);
    return hipDeviceSynchronize() == hipSuccess ? 0 : -1;
}
