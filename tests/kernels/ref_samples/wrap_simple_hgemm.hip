// Runs the device kernel of the reference's samples/simple_hgemm.cpp, compiled unchanged against
// this library's headers, with the sample's own launch geometry (samples/simple_hgemm.cpp:186-218).
// The sample's main() is renamed away; nothing else of the file is touched.
#define main sample_main_unused
#include "simple_hgemm.cpp"
#undef main

extern "C" int ref_simple_hgemm(uint32_t m, uint32_t n, uint32_t k, const void* a, const void* b, const void* c, void* d,
                                uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd, float alpha, float beta)
{
    const uint32_t wave = 64; // wave64 target
    auto blockDim = dim3(4 * wave, T_BLOCK_Y);
    auto gridDim  = dim3(rocwmma::ceilDiv(m, ROCWMMA_M * 4u), rocwmma::ceilDiv(n, ROCWMMA_N * T_BLOCK_Y));
    hipLaunchKernelGGL(hgemm_rocwmma_d, gridDim, blockDim, 0, 0, m, n, k, static_cast<const float16_t*>(a),
                       static_cast<const float16_t*>(b), static_cast<const float16_t*>(c), static_cast<float16_t*>(d), lda,
                       ldb, ldc, ldd, alpha, beta);
    return hipDeviceSynchronize() == hipSuccess ? 0 : -1;
}
