// Runs the device kernel of the reference's samples/perf_hgemm.cpp (cooperative global -> LDS staging,
// transforms, 2 x 2 blocks per wave), compiled unchanged against this library's headers, with the
// sample's wave64 launch geometry (samples/perf_hgemm.cpp:224-237, 807-842).
#define main sample_main_unused
#include "perf_hgemm.cpp"
#undef main

extern "C" int ref_perf_hgemm(uint32_t m, uint32_t n, uint32_t k, const void* a, const void* b, const void* c, void* d,
                              uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd, float alpha, float beta)
{
    namespace P = gfx9Params;
    const uint32_t macroX = (P::TBLOCK_X / 64u) * P::BLOCKS_X * P::ROCWMMA_M;
    const uint32_t macroY = P::TBLOCK_Y * P::BLOCKS_Y * P::ROCWMMA_N;
    auto blockDim = dim3(P::TBLOCK_X, P::TBLOCK_Y);
    auto gridDim  = dim3(rocwmma::ceilDiv(m, macroX), rocwmma::ceilDiv(n, macroY));
    const int lds = 2u * sizeof(InputT) * (macroX + macroY) * P::ROCWMMA_K;
    hipLaunchKernelGGL(gemm_rocwmma_d, gridDim, blockDim, lds, 0, m, n, k, static_cast<const InputT*>(a),
                       static_cast<const InputT*>(b), static_cast<const OutputT*>(c), static_cast<OutputT*>(d), lda, ldb,
                       ldc, ldd, alpha, beta);
    return hipDeviceSynchronize() == hipSuccess ? 0 : -1;
}
